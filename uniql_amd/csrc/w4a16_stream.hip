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
// Every byte of the 1 KiB row segment is fetched once, the codes are expanded to
// fp16 (code-8)*scale in registers exactly as the reference does, and eight MFMAs
// (one per jb) consume two packed rows (32 K values) at a time.  The activations
// are the A operand: rows of X (up to 16 per M-tile) staged through LDS in the same
// K order.  MFMA is used purely as a wide dot-product unit: its cost does not
// depend on M, so M = 1..16 all run at the weight-streaming rate.
//
// Work split: unit = (strip of 128 columns) x (group of 128 K).  A wave owns `upw`
// consecutive groups of a strip, the four waves of a workgroup own consecutive
// group ranges, partial sums meet in LDS.  When K is split over several workgroups
// they store fp32 partials; the last workgroup to arrive (a counter in `workspace`,
// which it resets to zero) adds them in a fixed order, so results are
// deterministic and no workgroup ever waits for another.
#include "common.hpp"

namespace uniql {

constexpr int kXsStride = 68;  // dwords per staged activation row: 64 + 4, keeps the 64 lanes on distinct banks

struct StreamArgs {
    const u32x4* B;       // packed weights, [K/16][N/2] 16-byte pieces
    const half_t* S;      // permuted scales [groups][N]
    const half_t* X;      // activations [M][ldx]
    void* D;              // fp16 or fp32 [M][N]
    float* partial;       // [splits][M][N] when splits > 1
    int32_t* counters;    // [N/128], zero on entry and on exit
    int64_t ldx;
    int M, N, K;
    int G;                // number of 128-wide K groups = K/128
    int per_column;       // 1: a single scale row (per-column scales)
    int upw;              // groups per wave
    int splits;           // workgroups along K per strip
    int out_f32;
    float had_scale;
};

// Registers: MT = 1 needs ~140 VGPRs, which allows 3 waves per SIMD (12 per CU, 96 KiB
// of weight loads in flight per CU); the bigger M tiles trade occupancy for accumulators.
template <int MT, bool HAD>
__global__ __launch_bounds__(256, (MT == 1 ? 3 : (MT == 2 ? 2 : 1))) void w4a16_stream_kernel(const StreamArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
    __shared__ int s_last;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int w = tid >> 6;
    const int slot = lane & 15;
    const int kq = lane >> 4;
    const int c8 = slot & 7;

    const int nstrips = a.N >> 7;
    const int strip = blockIdx.x % nstrips;
    const int split = blockIdx.x / nstrips;
    const int chunk = 2 * strip + (slot >> 3);

    const int N4 = a.N >> 1;  // 16-byte pieces per packed row
    const int g_begin = (split * 4 + w) * a.upw;

    f4 acc[MT][8];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int jb = 0; jb < 8; ++jb) acc[mt][jb] = f4{0.f, 0.f, 0.f, 0.f};

    uint32_t* xs = lds + (size_t)w * (MT * 16) * kXsStride;  // this wave's staging rows

    u32x4 wq[8];
    auto load_weights = [&](int g) {
        const u32x4* bp = a.B + (size_t)(8 * g) * N4 + chunk * 32 + 4 * c8 + kq;
#pragma unroll
        for (int rr = 0; rr < 8; ++rr) wq[rr] = __builtin_nontemporal_load(bp + (size_t)rr * N4);
    };

    for (int u = 0; u < a.upw; ++u) {
        const int g = g_begin + u;
        if (g >= a.G) break;  // wave-uniform

        // ---- activations X[:, 128g .. 128g+127]: issue the loads first ------------
        u32x4 xv[MT][4];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int m = mt * 16 + i * 4 + (lane >> 4);
                xv[mt][i] = u32x4{0u, 0u, 0u, 0u};
                if (m < a.M)
                    xv[mt][i] = *reinterpret_cast<const u32x4*>(a.X + (size_t)m * a.ldx + 128 * g + 8 * slot);
            }
        }

        // ---- scales of this lane's eight columns --------------------------------
        u32x4 sc;
        if (!a.per_column) {
            sc = *reinterpret_cast<const u32x4*>(a.S + (size_t)g * a.N + chunk * 64 + 8 * c8);
        } else {
            uint32_t t[4];
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const int n0 = chunk * 64 + c8 + 8 * (2 * p), n1 = n0 + 8;
                const uint16_t lo = *reinterpret_cast<const uint16_t*>(a.S + single_scale_pos(n0));
                const uint16_t hi = *reinterpret_cast<const uint16_t*>(a.S + single_scale_pos(n1));
                t[p] = (uint32_t)lo | ((uint32_t)hi << 16);
            }
            sc = u32x4{t[0], t[1], t[2], t[3]};
        }

        // the first group's weights go out behind the (small) activation loads, so
        // that staging overlaps the weight latency; later groups were prefetched
        if (u == 0) load_weights(g);

        // ---- rotate (optionally) and stage the activations in LDS ------------------
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                {
                    const int m = mt * 16 + i * 4 + (lane >> 4);
                    u32x4 v = xv[mt][i];
                    if (HAD) {
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
                            hv.x = (half_t)(f[2 * p] * a.had_scale);
                            hv.y = (half_t)(f[2 * p + 1] * a.had_scale);
                            v[p] = h2_to_bits(hv);
                        }
                    }
                    *reinterpret_cast<u32x4*>(xs + (size_t)m * kXsStride + 4 * slot) = v;
                }
            }
        }
        // LDS operations of one wave complete in issue order: the reads below see
        // the writes above without a workgroup barrier (each wave has its own rows).
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

        // keep the next group's weights in flight while this one is consumed
        u32x4 cur[8];
#pragma unroll
        for (int rr = 0; rr < 8; ++rr) cur[rr] = wq[rr];
        if (u + 1 < a.upw && g + 1 < a.G) load_weights(g + 1);

        h2 s2[8];
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const h2 pr = bits_to_h2(sc[p]);
            s2[2 * p] = h2{pr.x, pr.x};
            s2[2 * p + 1] = h2{pr.y, pr.y};
        }

#pragma unroll
        for (int rp = 0; rp < 4; ++rp) {
            h8 xa[MT];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const uint32_t* xr = xs + (size_t)(mt * 16 + slot) * kXsStride + 16 * rp + kq;
                const h2 d0 = bits_to_h2(xr[0]), d1 = bits_to_h2(xr[4]);
                const h2 d2 = bits_to_h2(xr[8]), d3 = bits_to_h2(xr[12]);
                xa[mt] = h8{d0.x, d0.y, d1.x, d1.y, d2.x, d2.y, d3.x, d3.y};
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t q0 = cur[2 * rp][j], q1 = cur[2 * rp + 1][j];
#pragma unroll
                for (int blk = 0; blk < 2; ++blk) {
                    const uint32_t p0 = blk ? (q0 >> 8) : q0;
                    const uint32_t p1 = blk ? (q1 >> 8) : q1;
                    const h2 sv = s2[2 * j + blk];
                    const h2 e0 = code_pair_low(p0) * sv, e1 = code_pair_high(p0) * sv;
                    const h2 e2 = code_pair_low(p1) * sv, e3 = code_pair_high(p1) * sv;
                    const h8 bw = h8{e0.x, e0.y, e1.x, e1.y, e2.x, e2.y, e3.x, e3.y};
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt)
                        acc[mt][2 * j + blk] =
                            __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[mt], bw, acc[mt][2 * j + blk], 0, 0, 0);
                }
            }
        }
    }

    // ---- combine the four waves, then the K splits ---------------------------------
    // acc[mt][jb][v] on lane l is row m = 16 mt + 4 (l/16) + v, column
    // 128 strip + 64 (slot/8) + 16 (jb/2) + 8 (jb%2) + slot%8.
    float* red = reinterpret_cast<float*>(lds);  // [4 waves][16 rows][128 columns]
    const int ncol_lane = 64 * (slot >> 3) + c8;
    const int col_out = tid & 127;
    const int n_out = 128 * strip + col_out;
    for (int mt = 0; mt < MT; ++mt) {
        if (mt * 16 >= a.M) break;
        __syncthreads();
#pragma unroll
        for (int jb = 0; jb < 8; ++jb) {
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int ml = 4 * kq + v;
                if (mt * 16 + ml < a.M)
                    red[(w * 16 + ml) * 128 + ncol_lane + 16 * (jb >> 1) + 8 * (jb & 1)] = acc[mt][jb][v];
            }
        }
        __syncthreads();
        for (int ml = tid >> 7; ml < 16; ml += 2) {
            const int m = mt * 16 + ml;
            if (m >= a.M) break;
            const float sum = (red[(0 * 16 + ml) * 128 + col_out] + red[(1 * 16 + ml) * 128 + col_out]) +
                              (red[(2 * 16 + ml) * 128 + col_out] + red[(3 * 16 + ml) * 128 + col_out]);
            if (a.splits == 1) {
                if (a.out_f32)
                    reinterpret_cast<float*>(a.D)[(size_t)m * a.N + n_out] = sum;
                else
                    reinterpret_cast<half_t*>(a.D)[(size_t)m * a.N + n_out] = (half_t)sum;
            } else {
                a.partial[((size_t)split * a.M + m) * a.N + n_out] = sum;
            }
        }
    }

    if (a.splits > 1) {
        __threadfence();
        __syncthreads();
        if (tid == 0) {
            const int prev = atomicAdd(a.counters + strip, 1);
            s_last = (prev == a.splits - 1);
        }
        __syncthreads();
        if (s_last) {
            __threadfence();
            for (int m = tid >> 7; m < a.M; m += 2) {
                float sum = 0.f;
                for (int sp = 0; sp < a.splits; ++sp)
                    sum += __builtin_nontemporal_load(a.partial + ((size_t)sp * a.M + m) * a.N + n_out);
                if (a.out_f32)
                    reinterpret_cast<float*>(a.D)[(size_t)m * a.N + n_out] = sum;
                else
                    reinterpret_cast<half_t*>(a.D)[(size_t)m * a.N + n_out] = (half_t)sum;
            }
            if (tid == 0) a.counters[strip] = 0;
        }
    }
}

// ---------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------
static inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

int stream_pick_upw(int n, int k) {
    const int nstrips = n / 128, G = k / 128;
    int upw = 1;
    while (upw < 8 && (int64_t)nstrips * ceil_div(G, 4 * upw) > 1024) upw *= 2;
    return upw;
}

size_t stream_partial_bytes(int m, int n, int k) {
    // worst case over the possible units-per-wave choices (upw = 1)
    const int G = k / 128;
    const int splits = ceil_div(G, 4);
    if (splits <= 1) return 0;
    const int mrows = m < 64 ? m : 64;
    return (size_t)splits * mrows * n * sizeof(float);
}

template <int MT, bool HAD>
static hipError_t launch_one(const StreamArgs& a, hipStream_t stream) {
    const size_t stage = (size_t)4 * MT * 16 * kXsStride * 4;
    const size_t red = (size_t)4 * 16 * 128 * 4;
    const size_t shmem = stage > red ? stage : red;
    if (shmem > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&w4a16_stream_kernel<MT, HAD>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
        if (e != hipSuccess) return e;
    }
    const int grid = (a.N / 128) * a.splits;
    hipLaunchKernelGGL((w4a16_stream_kernel<MT, HAD>), dim3(grid), dim3(256), shmem, stream, a);
    return hipGetLastError();
}

// Rows are processed in slabs of at most 64; every slab re-streams the weights.
int stream_launch(const void* A, int64_t lda, const void* B, const void* S, void* D, int32_t* workspace,
                  void* scratch, int m, int n, int k, int groups, bool had128, float had_scale, bool out_f32,
                  int upw_override, hipStream_t stream) {
    StreamArgs a;
    a.B = reinterpret_cast<const u32x4*>(B);
    a.S = reinterpret_cast<const half_t*>(S);
    a.partial = reinterpret_cast<float*>(scratch);
    a.counters = workspace;
    a.ldx = lda;
    a.N = n;
    a.K = k;
    a.G = k / 128;
    a.per_column = (groups == 1) ? 1 : 0;
    a.upw = upw_override > 0 ? upw_override : stream_pick_upw(n, k);
    a.splits = ceil_div(a.G, 4 * a.upw);
    a.out_f32 = out_f32 ? 1 : 0;
    a.had_scale = had_scale;
    const size_t out_elt = out_f32 ? 4 : 2;
    for (int m0 = 0; m0 < m; m0 += 64) {
        const int mm = (m - m0) < 64 ? (m - m0) : 64;
        a.M = mm;
        a.X = reinterpret_cast<const half_t*>(A) + (size_t)m0 * lda;
        a.D = reinterpret_cast<char*>(D) + (size_t)m0 * n * out_elt;
        hipError_t e;
        const int mt = ceil_div(mm, 16);
        if (had128) {
            if (mt == 1) e = launch_one<1, true>(a, stream);
            else if (mt == 2) e = launch_one<2, true>(a, stream);
            else e = launch_one<4, true>(a, stream);
        } else {
            if (mt == 1) e = launch_one<1, false>(a, stream);
            else if (mt == 2) e = launch_one<2, false>(a, stream);
            else e = launch_one<4, false>(a, stream);
        }
        if (e != hipSuccess) return UNIQL_E_LAUNCH;
    }
    return UNIQL_OK;
}

}  // namespace uniql
