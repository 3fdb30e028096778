// Large f32 matrix products C[M,N] = op(A) . op(B) with both operands staged through LDS in 64-deep slabs, for the
// shapes where the generic implicit-GEMM tile (16-deep slabs, one dword load per element) tops out near 64 % of the
// MFMA peak.  Same product as launch_matmul of the reference (src/backend/cuda/kernels.rs:919-938, cpu.rs:967-1002).
//
// A block (4 waves) owns a 128 x BN tile, BN = 32*TN (TN = 4 or 2): wave w owns rows [32w, 32w+32) and all BN columns,
// i.e. TN accumulator blocks of 32x32 (v_mfma_f32_32x32x2_f32).  Per stage (KC = 64 values of k) LDS holds both operand
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

constexpr int BM = 128, KC = 64, NT = 256;
constexpr int PK = KC + 1;  // pitch of a k-contiguous slab row
constexpr size_t LDS_BUDGET = 72 * 1024;

struct Params {
    const float* A;
    const float* B;
    float* C;
    const float* bias;  // optional, per column of C; with relu != 0 the sum is clamped at 0 afterwards
    int relu;
    int M, N, K;
    i64 lda, ldb;  // leading dimensions of the operands as stored
    int tiles_n, tiles, xcd_chunk;
};

// TA: A is stored [K, M] (m contiguous); TB: B is stored [N, K] (k contiguous).
template <int TN, bool TA, bool TB, bool BIAS>
__global__ __launch_bounds__(NT, 2) void gemm_lds_kernel(const Params p) {
    constexpr int BN = 32 * TN;
    constexpr int PA = TA ? BM : PK, PB = TB ? PK : BN;          // LDS pitches
    constexpr int ASZ = TA ? KC * BM : BM * PK, BSZ = TB ? BN * PK : KC * BN;
    constexpr int NA = BM * KC / 4 / NT, NB = BN * KC / 4 / NT;  // float4 per thread per stage
    static_assert(BN * KC % (4 * NT) == 0, "B slab must divide over the block");
    extern __shared__ __align__(16) float smem[];
    float* As = smem;
    float* Bs = smem + ASZ;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, l32 = lane & 31;

    // id -> tile: XCD x gets tiles [x * chunk, (x+1) * chunk) when the tile count divides by 8
    int tile = blockIdx.x;
    if (p.xcd_chunk) tile = (tile & 7) * p.xcd_chunk + (tile >> 3);
    const int tm = tile / p.tiles_n, tn = tile - tm * p.tiles_n;
    const int m0 = tm * BM, n0 = tn * BN;

    f32x16 acc[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j)
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
        const int c4 = min(m0 + 4 * (tid & 31), p.M - 4);
#pragma unroll
        for (int u = 0; u < NA; ++u) a_off[u] = (uint32_t)((i64)((tid >> 5) + 8 * u) * p.lda + c4) * 4u;
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
    auto prefetch = [&](int k0) {
        const float* a = TA ? p.A + (i64)k0 * p.lda : p.A + k0;
        const float* b = TB ? p.B + k0 : p.B + (i64)k0 * p.ldb;
#pragma unroll
        for (int u = 0; u < NA; ++u) av[u] = ldg4(a, a_off[u]);
#pragma unroll
        for (int u = 0; u < NB; ++u) bv[u] = ldg4(b, b_off[u]);
    };
    auto park = [&]() {
        int t = tid;
        asm volatile("" : "+v"(t));  // recompute the LDS addresses here instead of keeping them alive over the MFMA loop
        if (!TA) {
#pragma unroll
            for (int u = 0; u < NA; ++u) {
                float* d = As + ((t >> 4) + 16 * u) * PK + 4 * (t & 15);
                d[0] = av[u].x; d[1] = av[u].y; d[2] = av[u].z; d[3] = av[u].w;
            }
        } else {
#pragma unroll
            for (int u = 0; u < NA; ++u) *reinterpret_cast<float4*>(As + ((t >> 5) + 8 * u) * BM + 4 * (t & 31)) = av[u];
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
    const float* const ar = TA ? As + half * PA + wave * 32 + l32 : As + (wave * 32 + l32) * PA + half;
    const float* const br = TB ? Bs + l32 * PB + half : Bs + half * PB + l32;
    auto compute = [&]() {
        float a0, b0[TN], a1, b1[TN];
        auto rd = [&](float& a, float (&b)[TN], int s) {
            a = TA ? ar[2 * s * PA] : ar[2 * s];
#pragma unroll
            for (int j = 0; j < TN; ++j) b[j] = TB ? br[j * 32 * PB + 2 * s] : br[2 * s * PB + j * 32];
            __builtin_amdgcn_sched_barrier(0);
        };
        auto mma = [&](float a, const float (&b)[TN]) {
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b[j], acc[j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        };
        rd(a0, b0, 0);
#pragma unroll
        for (int s = 0; s < KC / 2; s += 2) {
            rd(a1, b1, s + 1);
            mma(a0, b0);
            if (s + 2 < KC / 2) rd(a0, b0, s + 2);
            mma(a1, b1);
        }
    };

    prefetch(0);
    park();
    __syncthreads();
    for (int k0 = 0; k0 < p.K; k0 += KC) {
        const bool more = k0 + KC < p.K;
        if (more) prefetch(k0 + KC);
        __builtin_amdgcn_s_setprio(3);  // a co-resident block that is staging must not delay these MFMAs
        compute();
        __builtin_amdgcn_s_setprio(0);
        __syncthreads();
        if (more) park();
        __syncthreads();
    }

#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int n = n0 + j * 32 + l32;
        const float bj = BIAS ? p.bias[n < p.N ? n : p.N - 1] : 0.f;
        if (n < p.N) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int m = m0 + wave * 32 + igemm::Mfma<float>::row(e, lane);
                if (m < p.M) {
                    float v = acc[j][e];
                    if (BIAS) {
                        v = v + bj;
                        if (p.relu) v = v > 0.f ? v : 0.f;
                    }
                    p.C[(i64)m * p.N + n] = v;
                }
            }
        }
    }
}

struct Plan {
    bool ok = false;
    int TN = 4, tiles_m = 0, tiles_n = 0;
    size_t smem = 0;
};

// Taken for products that fill the chip without a K split: K a multiple of the 64-deep slab, 16-byte aligned rows,
// row-contiguous operands with a multiple of 4 rows, every byte offset inside a tile below 4 GiB.
inline Plan make_plan(int num_cus, bool ta, bool tb, i64 M, i64 N, i64 K, i64 lda, i64 ldb) {
    Plan pl;
    if (K < 2 * KC || K % KC != 0 || lda % 4 != 0 || ldb % 4 != 0 || M < BM || N < 64) return pl;
    if ((ta && M % 4 != 0) || (!tb && N % 4 != 0)) return pl;
    // tile width: the one with the least (rounds of co-resident blocks) x (work of a block); a nearly empty last round
    // costs as much as a full one (3072 x 3072: 576 tiles of 128 x 128 take two rounds, 1152 of 128 x 64 take 2.25)
    pl.tiles_m = (int)fx::ceil_div(M, (i64)BM);
    const i64 slots = 2 * (i64)std::max(1, num_cus);
    i64 best = -1, tiles = 0;
    for (int tn : {4, 2}) {
        const i64 t = (i64)pl.tiles_m * fx::ceil_div(N, (i64)(32 * tn));
        if (t < slots * 3 / 4) continue;  // fewer tiles: the generic kernel splits K instead
        const i64 cost = fx::ceil_div(t, slots) * tn * (tn == 2 ? 9 : 8);  // the narrow tile reads more per MFMA
        if (best < 0 || cost < best) {
            best = cost;
            pl.TN = tn;
            tiles = t;
        }
    }
    if (best < 0 || tiles > 0x7fffffff) return pl;
    pl.tiles_n = (int)fx::ceil_div(N, (i64)(32 * pl.TN));
    const i64 a_span = ta ? (i64)KC * lda + M : (i64)M * lda, b_span = tb ? (i64)N * ldb : (i64)KC * ldb + N;
    if (a_span * 4 >= (1ll << 32) || b_span * 4 >= (1ll << 32)) return pl;
    const int bn = 32 * pl.TN;
    pl.smem = (size_t)((ta ? KC * BM : BM * PK) + (tb ? bn * PK : KC * bn)) * sizeof(float);
    if (pl.smem > LDS_BUDGET) return pl;
    pl.ok = true;
    return pl;
}

template <int TN, bool TA, bool TB>
inline int launch(fx_ctx* c, const Plan& pl, const Params& p) {
    const dim3 grid((unsigned)p.tiles), blk(NT);
    static const hipError_t attr0 = hipFuncSetAttribute((const void*)gemm_lds_kernel<TN, TA, TB, false>,
                                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_BUDGET);
    static const hipError_t attr1 = hipFuncSetAttribute((const void*)gemm_lds_kernel<TN, TA, TB, true>,
                                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_BUDGET);
    FX_HIP_CHECK(attr0);
    FX_HIP_CHECK(attr1);
    if (p.bias) gemm_lds_kernel<TN, TA, TB, true><<<grid, blk, pl.smem, c->stream>>>(p);
    else gemm_lds_kernel<TN, TA, TB, false><<<grid, blk, pl.smem, c->stream>>>(p);
    FX_LAUNCH_CHECK();
    return FX_OK;
}
template <bool TA, bool TB>
inline int launch_tn(fx_ctx* c, const Plan& pl, const Params& p) {
    return pl.TN == 4 ? launch<4, TA, TB>(c, pl, p) : launch<2, TA, TB>(c, pl, p);
}

// A, B and C must be 16-byte aligned.
inline int run(fx_ctx* c, const Plan& pl, bool ta, bool tb, i64 M, i64 N, i64 K, const float* A, const float* B, float* C,
               const float* bias, int relu) {
    Params p;
    p.A = A; p.B = B; p.C = C; p.bias = bias; p.relu = relu;
    p.M = (int)M; p.N = (int)N; p.K = (int)K;
    p.lda = ta ? M : K;
    p.ldb = tb ? K : N;
    p.tiles_n = pl.tiles_n;
    p.tiles = pl.tiles_m * pl.tiles_n;
    p.xcd_chunk = p.tiles % 8 == 0 ? p.tiles / 8 : 0;
    if (!ta && !tb) return launch_tn<false, false>(c, pl, p);
    if (!ta && tb) return launch_tn<false, true>(c, pl, p);
    if (ta && !tb) return launch_tn<true, false>(c, pl, p);
    return launch_tn<true, true>(c, pl, p);
}

}  // namespace glk
