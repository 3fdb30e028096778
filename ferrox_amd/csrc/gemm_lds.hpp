// Large f32 matrix products C[M,N] = op(A) . op(B) with both operands staged through LDS in 64-deep slabs, for the
// shapes where the generic implicit-GEMM tile (16-deep slabs, one dword load per element) tops out near 64 % of the
// MFMA peak.  Same product as launch_matmul of the reference (src/backend/cuda/kernels.rs:919-938, cpu.rs:967-1002).
//
// A block (4 waves) owns a BM x BN tile, BM = 32*WM, BN = 32*TN*(4/WM): the waves are laid out WM x (4/WM); a wave owns 32
// rows and 32*TN columns, i.e. TN accumulator blocks of 32x32 (v_mfma_f32_32x32x2_f32).  Large products take 128 x 128 or
// 128 x 64 tiles (WM = 4, TN = 4 or 2); products with too few of those to fill the chip (1024^3: 64 tiles) take 64 x 128 or
// 64 x 64 tiles (WM = 2, TN = 2 or 1) instead of a K split with partial sums in memory; with one accumulator block per wave
// the even and the odd MFMA steps add into two accumulators (added once at the end), so that no MFMA waits for the one
// before it.  Per stage (KC = 64 values of k) LDS holds both operand
// slabs in the form their memory layout gives for free:
//   k-contiguous operand (A as stored [M,K]; B given as [N,K]):  S[r][k], pitch 65  -> the 32 lanes of an MFMA operand
//                                                               read (r = lane % 32, k + lane / 32) hit 32 banks
//   row-contiguous operand (A given as [K,M]; B as stored [K,N]): S[k][r], pitch 128 / BN -> lanes read 32 consecutive floats
// so staging is a straight copy of 16-byte global loads (four 4-byte LDS stores for the odd pitch, one 16-byte store
// otherwise) and the MFMA loop contains nothing but LDS reads with compile-time offsets.  The next stage's global
// loads are issued before the MFMA loop of the current stage and parked in registers; two blocks share a CU.
// Workgroup ids are handed to the eight XCDs round-robin by the hardware; the id -> tile map gives each XCD a
// contiguous range of tiles so that the tiles resident on one XCD share operand panels in its L2.
#pragma once
#include "igemm_core.hpp"

namespace glk {
using igemm::f32x16;
using igemm::ldg4;

constexpr int KC = 64, NT = 256;
constexpr int PK = KC + 1;  // pitch of a k-contiguous slab row
constexpr size_t LDS_BUDGET = 72 * 1024;       // one stage of the 128-row tiles: two blocks per CU
constexpr size_t LDS_BUDGET_MID = 104 * 1024;  // two stages of the 64-row tiles (one block per CU has to overlap by itself)

struct Params {
    const float* A;
    const float* B;
    float* C;
    const float* bias;  // optional, per column of C; with relu != 0 the sum is clamped at 0 afterwards
    int relu;
    int M, N, K;
    i64 lda, ldb;  // leading dimensions of the operands as stored
    int tiles_n, tiles, xcd_chunk;
    // a batch of independent products of one shape in one launch (blockIdx.y): element strides between them (0: shared operand)
    i64 sa = 0, sb = 0, sc = 0;
    int bias_per_row = 0;  // the bias belongs to the rows of C (a convolution's output channels) instead of its columns
};

// TA: A is stored [K, M] (m contiguous); TB: B is stored [N, K] (k contiguous).
// KT (both operands k-contiguous only): K need not be a multiple of the stage depth -- the last stage loads what is left of the rows
// (K a multiple of 4: a 16-byte vector is inside a row or past it) and parks zeros behind it.
template <int TN, int WM, bool TA, bool TB, bool BIAS, bool KT = false>
__global__ __launch_bounds__(NT, 2) void gemm_lds_kernel(const Params p) {
    static_assert(!KT || (!TA && TB), "the K tail is handled for k-contiguous operands");
    constexpr int WN = 4 / WM, BM = 32 * WM, BN = 32 * TN * WN;
    constexpr int NACC = TN == 1 ? 2 : TN;  // accumulator blocks of a wave (TN == 1: even and odd MFMA steps apart)
    // The 128-row tiles keep one stage in LDS and rely on the CU's second block to cover staging; the 64-row tiles run where
    // there is about one block per CU, so they keep two stages: the next stage is parked while other waves still compute and a
    // stage costs one barrier.
    constexpr int STAGES = WM == 2 ? 2 : 1;
    constexpr int PA = TA ? BM : PK, PB = TB ? PK : BN;          // LDS pitches
    constexpr int ASZ = TA ? KC * BM : BM * PK, BSZ = TB ? BN * PK : KC * BN;
    constexpr int NA = BM * KC / 4 / NT, NB = BN * KC / 4 / NT;  // float4 per thread per stage
    static_assert(BN * KC % (4 * NT) == 0, "B slab must divide over the block");
    FX_DYNAMIC_SMEM(float, smem);
    float* As = smem;
    float* Bs = smem + ASZ;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, l32 = lane & 31;
    const int wm = wave % WM, wn = wave / WM;
    const float* const Ab = p.A + (i64)blockIdx.y * p.sa;
    const float* const Bb = p.B + (i64)blockIdx.y * p.sb;
    float* const Cb = p.C + (i64)blockIdx.y * p.sc;

    // id -> tile: XCD x gets tiles [x * chunk, (x+1) * chunk) when the tile count divides by 8
    int tile = blockIdx.x;
    if (p.xcd_chunk) tile = (tile & 7) * p.xcd_chunk + (tile >> 3);
    const int tm = tile / p.tiles_n, tn = tile - tm * p.tiles_n;
    const int m0 = tm * BM, n0 = tn * BN;

    f32x16 acc[NACC];
#pragma unroll
    for (int j = 0; j < NACC; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[j][e] = 0.f;

    // staging maps.  k-contiguous slab: thread t owns float4 column t % 16 (k = 4*(t%16)..+3) of rows t/16 + 16u.
    // row-contiguous slab of R floats per k: thread t owns float4 column t % (R/4) of k rows t/(R/4) + (NT/(R/4))u.
    uint32_t a_off[NA], b_off[NB];
    if (!TA) {
#pragma unroll
        for (int u = 0; u < NA; ++u) {
            const int r = min(m0 + (tid >> 4) + 16 * u, p.M - 1);  // rows past the matrix re-read its last row
            a_off[u] = (uint32_t)((i64)r * p.lda + 4 * (tid & 15)) * 4u;
        }
    } else {
        constexpr int Q = BM / 4, RS = NT / Q;  // float4 per k row, k rows per pass
        const int c4 = min(m0 + 4 * (tid % Q), p.M - 4);
#pragma unroll
        for (int u = 0; u < NA; ++u) a_off[u] = (uint32_t)((i64)(tid / Q + RS * u) * p.lda + c4) * 4u;
    }
    if (TB) {
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            const int r = min(n0 + (tid >> 4) + 16 * u, p.N - 1);
            b_off[u] = (uint32_t)((i64)r * p.ldb + 4 * (tid & 15)) * 4u;
        }
    } else {
        constexpr int Q = BN / 4, RS = NT / Q;  // float4 per k row, k rows per pass
        const int c4 = min(n0 + 4 * (tid % Q), p.N - 4);
#pragma unroll
        for (int u = 0; u < NB; ++u) b_off[u] = (uint32_t)((i64)(tid / Q + RS * u) * p.ldb + c4) * 4u;
    }
    float4 av[NA], bv[NB];
    bool dead = false;  // KT: this thread's four k of the stage in flight lie past K (its loads re-read the stage's first vector)
    auto prefetch = [&](int k0) {
        const float* a = TA ? Ab + (i64)k0 * p.lda : Ab + k0;
        const float* b = TB ? Bb + k0 : Bb + (i64)k0 * p.ldb;
        uint32_t back = 0;
        if constexpr (KT) {
            dead = k0 + 4 * (tid & 15) >= p.K;
            back = dead ? 16u * (tid & 15) : 0u;
        }
#pragma unroll
        for (int u = 0; u < NA; ++u) av[u] = ldg4(a, a_off[u] - back);
#pragma unroll
        for (int u = 0; u < NB; ++u) bv[u] = ldg4(b, b_off[u] - back);
    };
    auto park = [&](int buf) {
        int t = tid;
        FX_PIN_VGPR(t);  // recompute the LDS addresses here instead of keeping them alive over the MFMA loop
        float* const As = smem + buf * (ASZ + BSZ);
        float* const Bs = As + ASZ;
        if constexpr (KT) {
            if (dead) {
#pragma unroll
                for (int u = 0; u < NA; ++u) av[u] = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
                for (int u = 0; u < NB; ++u) bv[u] = make_float4(0.f, 0.f, 0.f, 0.f);
            }
        }
        if (!TA) {
#pragma unroll
            for (int u = 0; u < NA; ++u) {
                float* d = As + ((t >> 4) + 16 * u) * PK + 4 * (t & 15);
                d[0] = av[u].x; d[1] = av[u].y; d[2] = av[u].z; d[3] = av[u].w;
            }
        } else {
            constexpr int Q = BM / 4, RS = NT / Q;
#pragma unroll
            for (int u = 0; u < NA; ++u) *reinterpret_cast<float4*>(As + (t / Q + RS * u) * BM + 4 * (t % Q)) = av[u];
        }
        if (TB) {
#pragma unroll
            for (int u = 0; u < NB; ++u) {
                float* d = Bs + ((t >> 4) + 16 * u) * PK + 4 * (t & 15);
                d[0] = bv[u].x; d[1] = bv[u].y; d[2] = bv[u].z; d[3] = bv[u].w;
            }
        } else {
            constexpr int Q = BN / 4, RS = NT / Q;
#pragma unroll
            for (int u = 0; u < NB; ++u) *reinterpret_cast<float4*>(Bs + (t / Q + RS * u) * BN + 4 * (t % Q)) = bv[u];
        }
    };

    // operand reads of MFMA step s (k = 2s, 2s+1; lane half h takes k = 2s + h)
    const float* const ar = TA ? As + half * PA + wm * 32 + l32 : As + (wm * 32 + l32) * PA + half;
    const float* const br = TB ? Bs + (wn * 32 * TN + l32) * PB + half : Bs + half * PB + wn * 32 * TN + l32;
    auto compute = [&](int buf) {
        float a0, b0[TN], a1, b1[TN];
        const float* const arb = ar + buf * (ASZ + BSZ);
        const float* const brb = br + buf * (ASZ + BSZ);
        auto rd = [&](float& a, float (&b)[TN], int s) {
            a = TA ? arb[2 * s * PA] : arb[2 * s];
#pragma unroll
            for (int j = 0; j < TN; ++j) b[j] = TB ? brb[j * 32 * PB + 2 * s] : brb[2 * s * PB + j * 32];
            __builtin_amdgcn_sched_barrier(0);
        };
        auto mma = [&](float a, const float (&b)[TN], int parity) {
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int q = TN == 1 ? parity : j;
                acc[q] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b[j], acc[q], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        };
        if constexpr (STAGES == 2) {
            // one block per CU, one wave per SIMD: the operand reads run two MFMA steps ahead (three register sets), which
            // covers the LDS latency that a second wave would otherwise hide
            float a2, b2[TN];
            rd(a0, b0, 0);
            rd(a1, b1, 1);
#pragma unroll
            for (int s = 0; s < KC / 2; s += 6) {
                if (s + 2 < KC / 2) rd(a2, b2, s + 2);
                mma(a0, b0, 0);
                if (s + 3 < KC / 2) rd(a0, b0, s + 3);
                mma(a1, b1, 1);
                if (s + 2 < KC / 2) {
                    if (s + 4 < KC / 2) rd(a1, b1, s + 4);
                    mma(a2, b2, 0);
                }
                if (s + 3 < KC / 2) {
                    if (s + 5 < KC / 2) rd(a2, b2, s + 5);
                    mma(a0, b0, 1);
                }
                if (s + 4 < KC / 2) {
                    if (s + 6 < KC / 2) rd(a0, b0, s + 6);
                    mma(a1, b1, 0);
                }
                if (s + 5 < KC / 2) {
                    if (s + 7 < KC / 2) rd(a1, b1, s + 7);
                    mma(a2, b2, 1);
                }
            }
        } else {
            rd(a0, b0, 0);
#pragma unroll
            for (int s = 0; s < KC / 2; s += 2) {
                rd(a1, b1, s + 1);
                mma(a0, b0, 0);
                if (s + 2 < KC / 2) rd(a0, b0, s + 2);
                mma(a1, b1, 1);
            }
        }
    };

    prefetch(0);
    park(0);
    __syncthreads();
    if constexpr (STAGES == 1) {
        for (int k0 = 0; k0 < p.K; k0 += KC) {
            const bool more = k0 + KC < p.K;
            if (more) prefetch(k0 + KC);
            __builtin_amdgcn_s_setprio(3);  // a co-resident block that is staging must not delay these MFMAs
            compute(0);
            __builtin_amdgcn_s_setprio(0);
            __syncthreads();
            if (more) park(0);
            __syncthreads();
        }
    } else {
        int cur = 0;
        for (int k0 = 0; k0 < p.K; k0 += KC) {
            const bool more = k0 + KC < p.K;
            if (more) prefetch(k0 + KC);
            compute(cur);
            // the other buffer was last read in the stage before this one, which every wave has left through the barrier below
            if (more) park(cur ^ 1);
            __syncthreads();
            cur ^= 1;
        }
    }

    if constexpr (TN == 1) {
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[0][e] = acc[0][e] + acc[1][e];
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int n = n0 + (wn * TN + j) * 32 + l32;
        const float bj = BIAS && !p.bias_per_row ? p.bias[n < p.N ? n : p.N - 1] : 0.f;
        if (n < p.N) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int m = m0 + wm * 32 + igemm::Mfma<float>::row(e, lane);
                if (m < p.M) {
                    float v = acc[j][e];
                    if (BIAS) {
                        v = v + (p.bias_per_row ? p.bias[m] : bj);
                        if (p.relu) v = v > 0.f ? v : 0.f;
                    }
                    Cb[(i64)m * p.N + n] = v;
                }
            }
        }
    }
}

struct Plan {
    bool ok = false;
    int TN = 4, WM = 4, tiles_m = 0, tiles_n = 0;
    size_t smem = 0;
    int bm() const { return 32 * WM; }
    int bn() const { return 32 * TN * (4 / WM); }
};

// Taken for products that fill the chip without a K split: K a multiple of the 64-deep slab, 16-byte aligned rows,
// row-contiguous operands with a multiple of 4 rows, every byte offset inside a tile below 4 GiB.  batch: independent
// products of this shape that share the launch (their tiles count towards filling the chip).
inline Plan make_plan(int num_cus, bool ta, bool tb, i64 M, i64 N, i64 K, i64 lda, i64 ldb, i64 batch = 1) {
    Plan pl;
    // (a K that is no multiple of the stage depth: only with both operands k-contiguous, see KT in the kernel)
    if (K < 2 * KC || (K % KC != 0 && !(K % 4 == 0 && !ta && tb)) || lda % 4 != 0 || ldb % 4 != 0 || M < 64 || N < 64) return pl;
    if ((ta && M % 4 != 0) || (!tb && N % 4 != 0)) return pl;
    // tile shape: the one with the least (rounds of co-resident blocks) x (work of a block); a nearly empty last round
    // costs as much as a full one (3072 x 3072: 576 tiles of 128 x 128 take two rounds, 1152 of 128 x 64 take 2.25).  The
    // work of a block is its MFMA count weighted by what the tile reads per MFMA (narrower tiles re-read more).
    const i64 slots = 2 * (i64)std::max(1, num_cus);
    static const int shapes[4][3] = {{4, 4, 8}, {4, 2, 9}, {2, 2, 10}, {2, 1, 11}};  // WM, TN, cost per 32 x 32 block
    i64 best = -1, tiles = 0;
    for (const auto& sh : shapes) {
        const int wmv = sh[0], tn = sh[1], bm = 32 * wmv, bn = 32 * tn * (4 / wmv);
        if (M < bm) continue;
        const i64 t = fx::ceil_div(M, (i64)bm) * fx::ceil_div(N, (i64)bn) * batch;
        // fewer tiles than 3/4 of the block slots: a smaller tile, or (below half a block per CU even with the smallest)
        // the generic kernel's K split
        if (wmv == 4 ? t < slots * 3 / 4 : t < slots / 4) continue;
        const i64 cost = fx::ceil_div(t, slots) * (bm / 32) * (bn / 32) * sh[2];
        if (best < 0 || cost < best) {
            best = cost;
            pl.TN = tn;
            pl.WM = wmv;
            tiles = t;
        }
    }
    if (best < 0 || tiles > 0x7fffffff || batch > 65535) return pl;
    pl.tiles_m = (int)fx::ceil_div(M, (i64)pl.bm());
    pl.tiles_n = (int)fx::ceil_div(N, (i64)pl.bn());
    const i64 a_span = ta ? (i64)KC * lda + M : (i64)M * lda, b_span = tb ? (i64)N * ldb : (i64)KC * ldb + N;
    if (a_span * 4 >= (1ll << 32) || b_span * 4 >= (1ll << 32)) return pl;
    pl.smem = (size_t)((ta ? KC * pl.bm() : pl.bm() * PK) + (tb ? pl.bn() * PK : KC * pl.bn())) * sizeof(float) * (pl.WM == 2 ? 2 : 1);
    if (pl.smem > (pl.WM == 2 ? LDS_BUDGET_MID : LDS_BUDGET)) return pl;
    pl.ok = true;
    return pl;
}

template <int TN, int WM, bool TA, bool TB, bool KT = false>
inline int launch(fx_ctx* c, const Plan& pl, const Params& p, int batch) {
    const dim3 grid((unsigned)p.tiles, (unsigned)batch), blk(NT);
    if constexpr (!KT && !TA && TB) {
        if (p.K % KC != 0) return launch<TN, WM, TA, TB, true>(c, pl, p, batch);
    }
    static const hipError_t attr0 = hipFuncSetAttribute((const void*)gemm_lds_kernel<TN, WM, TA, TB, false, KT>,
                                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)(WM == 2 ? LDS_BUDGET_MID : LDS_BUDGET));
    static const hipError_t attr1 = hipFuncSetAttribute((const void*)gemm_lds_kernel<TN, WM, TA, TB, true, KT>,
                                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)(WM == 2 ? LDS_BUDGET_MID : LDS_BUDGET));
    FX_HIP_CHECK(attr0);
    FX_HIP_CHECK(attr1);
    if (p.bias) FX_LAUNCH(grid, blk, pl.smem, c->stream, (p), gemm_lds_kernel<TN, WM, TA, TB, true, KT>);
    else FX_LAUNCH(grid, blk, pl.smem, c->stream, (p), gemm_lds_kernel<TN, WM, TA, TB, false, KT>);
    FX_LAUNCH_CHECK();
    return FX_OK;
}
template <bool TA, bool TB>
inline int launch_tn(fx_ctx* c, const Plan& pl, const Params& p, int batch) {
    if (pl.WM == 4) return pl.TN == 4 ? launch<4, 4, TA, TB>(c, pl, p, batch) : launch<2, 4, TA, TB>(c, pl, p, batch);
    return pl.TN == 2 ? launch<2, 2, TA, TB>(c, pl, p, batch) : launch<1, 2, TA, TB>(c, pl, p, batch);
}

// A, B and C must be 16-byte aligned.  batch > 1: `batch` products in one launch, operand / result k of the batch sa / sb / sc
// elements after the first (a stride of 0 shares the operand); bias_per_row: the bias is indexed by the row of C.
inline int run(fx_ctx* c, const Plan& pl, bool ta, bool tb, i64 M, i64 N, i64 K, const float* A, const float* B, float* C,
               const float* bias, int relu, i64 batch = 1, i64 sa = 0, i64 sb = 0, i64 sc = 0, int bias_per_row = 0) {
    Params p;
    p.A = A; p.B = B; p.C = C; p.bias = bias; p.relu = relu;
    p.M = (int)M; p.N = (int)N; p.K = (int)K;
    p.lda = ta ? M : K;
    p.ldb = tb ? K : N;
    p.tiles_n = pl.tiles_n;
    p.tiles = pl.tiles_m * pl.tiles_n;
    p.xcd_chunk = p.tiles % 8 == 0 ? p.tiles / 8 : 0;
    p.sa = sa; p.sb = sb; p.sc = sc; p.bias_per_row = bias_per_row;
    if (!ta && !tb) return launch_tn<false, false>(c, pl, p, (int)batch);
    if (!ta && tb) return launch_tn<false, true>(c, pl, p, (int)batch);
    if (ta && !tb) return launch_tn<true, false>(c, pl, p, (int)batch);
    return launch_tn<true, true>(c, pl, p, (int)batch);
}

}  // namespace glk
