// Weight gradient of a 3x3 convolution (f32) with both operands staged in LDS in their natural layouts.
//
// dw[oc][c][ky][kx] = sum over (b, oy, ox) of g[b][oc][oy][ox] * x[b][c][oy*sh+ky-ph][ox*sw+kx-pw]
// (the product the reference forms as grad_out_2d . im2col(x)^T, src/backend/storage/extensions/convolutions.rs:296-338).
//
// One stage = R output rows of one image.  A block copies, per stage,
//   Gs[oc][pixel]      BM output-channel rows of g, pixels contiguous as in memory  (pitch GP,    GP % 32 == 4)
//   Xs[c][row][col]    32 input-channel planes of the zero-padded rows those pixels touch (pitch PLANE % 32 == 1)
// and every wave then runs 9 accumulator blocks of 32(oc) x 32(c), one per filter tap: the MFMA A operand of lane l
// is Gs[oc = l%32][pixel + l/32], the B operand of tap (ky,kx) is Xs[c = l%32][that pixel shifted by (ky,kx)].
// The odd plane pitch puts the 32 lanes of a half-wave on 32 different LDS banks for the nine B reads of a step;
// the single A read takes a 4-way conflict in exchange for 16-byte aligned rows (one 128-bit LDS store per
// float4 of g).  The patch is loaded once and serves all nine taps, so no im2col gather or bounds test is left
// in the MFMA loop.
// The pixel range is split over blockIdx.z into partial sums kept tap-major ([oc][tap][c], coalesced stores);
// a second kernel adds the partials in split order and writes dw in its [oc][c][tap] order.
#pragma once
#include "igemm_core.hpp"

namespace wgp {
using igemm::FastDiv;
using igemm::f32x16;


constexpr int KH = 3, KW = 3, KK = 9, CT = 32;  // filter taps; input channels per block
constexpr size_t LDS_BUDGET = 72 * 1024;        // per block, so that two blocks share a CU
constexpr int SLACK = 64;                       // floats behind the last plane that the look-ahead read may touch

// 16-byte load from global memory at a wave-uniform base plus a 32-bit byte offset (never a FLAT access, so it
// does not tie up the LDS counter that the MFMA loop waits on).
__device__ __forceinline__ float4 ldg4(const float* base, uint32_t byteoff) {
    typedef __attribute__((address_space(1))) const char gchar;
    typedef float v4 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(1))) const v4 gv4;
    const v4 v = *(gv4*)((gchar*)base + byteoff);
    return make_float4(v.x, v.y, v.z, v.w);
}

struct Params {
    const float* x;
    const float* g;
    float* part;
    int Cin, H, W, Cout, oh, ow, sh, sw, ph, pw;
    int R, PR, PW, PLANE, GP, Kst;  // rows per stage, patch rows/width, plane pitch, g pitch, pixels per stage
    int stages, sps, spi;           // all stages, stages per split, stages per image
    FastDiv div_spi, div_g4, div_xc, div_xr, div_kst, div_xcs, div_xrs;
    i64 part_stride;
};


constexpr int LPR = 16;  // lanes that share one row of a staged operand in the prefetching variant

// XR > 0 selects the prefetching variant: the next stage's global loads are issued before the MFMA loop of the
// current stage and held in registers until that loop is done.  It needs WM == 4, VEC, rows of at most
// 4*LPR floats (Kst <= 64, W <= 64) and exactly XR patch rows; thread t then owns float4 column t % 16 of rows
// t/16 + 16u, so every address is a per-thread constant plus a wave-uniform step and a stage costs a handful of
// vector instructions outside the MFMAs.  XR == 0: a stage is loaded, stored to LDS, then used.
template <int WM, bool VEC, int XR>
__global__ __launch_bounds__(64 * WM, 2) void wgrad_patch_kernel(const Params p) {
    constexpr bool PREF = XR > 0;
    static_assert(!PREF || (VEC && WM == 4), "prefetch needs the vector path and 256 threads");
    constexpr int NT = 64 * WM, BM = 32 * WM;
    constexpr int RPP = NT / LPR;                     // rows covered by one pass of the block
    constexpr int NG = BM / RPP, NXC = CT / RPP, NX = NXC * (PREF ? XR : 1);
    extern __shared__ __align__(16) float smem[];
    float* Gs = smem;
    float* Xs = smem + BM * p.GP;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, l32 = lane & 31;
    const int c0 = blockIdx.x * CT, oc0 = blockIdx.y * BM;
    const int L = p.oh * p.ow;
    const int k4 = p.Kst >> 2, w4 = p.W >> 2;
    const int ng4 = BM * k4, nx4 = CT * p.PR * w4;

    for (int i = tid; i < CT * p.PLANE + SLACK; i += NT) Xs[i] = 0.f;  // the padding columns stay zero from here on
    f32x16 acc[KK];
#pragma unroll
    for (int t = 0; t < KK; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[t][e] = 0.f;
    __syncthreads();

    const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
    auto stage_ptrs = [&](int s, const float*& gsrc, const float*& xsrc, int& iy0) {
        const int b = (int)p.div_spi.div((uint32_t)s);
        const int oy0 = (s - b * p.spi) * p.R;
        iy0 = oy0 * p.sh - p.ph;
        gsrc = p.g + ((i64)b * p.Cout + oc0) * L + (i64)oy0 * p.ow;
        xsrc = p.x + ((i64)b * p.Cin + c0) * p.H * p.W;
    };

    // ---- prefetching variant: registers of the stage in flight and the per-thread constants of its addresses
    float4 gv[PREF ? NG : 1], xv[PREF ? NX : 1];
    const int pq = tid & (LPR - 1), prow = tid / LPR;
    const bool g_lane = pq < k4, x_lane = pq < w4;
    const bool full_m = oc0 + BM <= p.Cout;
    const uint32_t g_off = g_lane ? (uint32_t)(prow * L + 4 * pq) * 4u : 0u;
    const uint32_t x_off = x_lane ? (uint32_t)(prow * p.H * p.W + 4 * pq) * 4u : 0u;
    const int g_dst0 = prow * p.GP + 4 * pq;
    const int x_dst0 = BM * p.GP + prow * p.PLANE + p.pw + 4 * pq;
    uint32_t x_rows = 0;  // bit r: patch row r of the stage in flight lies inside the image
    auto prefetch = [&](int s) {
        const float *gsrc, *xsrc;
        int iy0;
        stage_ptrs(s, gsrc, xsrc, iy0);
#pragma unroll
        for (int u = 0; u < NG; ++u) {
            const bool ok = full_m || oc0 + prow + u * RPP < p.Cout;
            gv[PREF ? u : 0] = ldg4(gsrc + (i64)u * RPP * L, ok ? g_off : 0u);
        }
        x_rows = 0;
#pragma unroll
        for (int r = 0; r < XR; ++r) {
            const int iy = iy0 + r;
            if (iy >= 0 && iy < p.H) {  // wave-uniform
                x_rows |= 1u << r;
#pragma unroll
                for (int cu = 0; cu < NXC; ++cu)
                    xv[PREF ? r * NXC + cu : 0] = ldg4(xsrc + ((i64)cu * RPP * p.H + iy) * p.W, x_off);
            }
        }
    };
    auto park = [&]() {
        int gd = g_dst0, xd = x_dst0;
        asm volatile("" : "+v"(gd), "+v"(xd));  // recompute the row addresses here instead of keeping 14 of them alive
        float* const g_dst = smem + gd;
        float* const x_dst = smem + xd;
        if (g_lane) {
#pragma unroll
            for (int u = 0; u < NG; ++u) {
                const bool ok = full_m || oc0 + prow + u * RPP < p.Cout;
                const float4 v = ok ? gv[PREF ? u : 0] : zero4;
                float* d = g_dst + u * RPP * p.GP;
                d[0] = v.x; d[1] = v.y; d[2] = v.z; d[3] = v.w;
            }
        }
        if (x_lane) {
#pragma unroll
            for (int r = 0; r < XR; ++r) {
                const bool ok = (x_rows >> r) & 1;  // wave-uniform
#pragma unroll
                for (int cu = 0; cu < NXC; ++cu) {
                    const float4 v = ok ? xv[PREF ? r * NXC + cu : 0] : zero4;
                    float* d = x_dst + cu * RPP * p.PLANE + r * p.PW;
                    d[0] = v.x; d[1] = v.y; d[2] = v.z; d[3] = v.w;
                }
            }
        }
    };

    // ---- plain variant
    auto stage_direct = [&](int s) {
        const float *gsrc, *xsrc;
        int iy0;
        stage_ptrs(s, gsrc, xsrc, iy0);
        if constexpr (VEC) {
            for (int i = tid; i < ng4; i += NT) {
                const int row = (int)p.div_g4.div((uint32_t)i), q = i - row * k4;
                const float4 v = oc0 + row < p.Cout ? ldg4(gsrc, (uint32_t)(row * L + 4 * q) * 4u) : zero4;
                float* d = Gs + row * p.GP + 4 * q;
                d[0] = v.x; d[1] = v.y; d[2] = v.z; d[3] = v.w;
            }
            for (int i = tid; i < nx4; i += NT) {
                const int c = (int)p.div_xc.div((uint32_t)i), rem = i - c * (p.PR * w4);
                const int r = (int)p.div_xr.div((uint32_t)rem), q = rem - r * w4;
                const int iy = iy0 + r;
                const float4 v = iy >= 0 && iy < p.H ? ldg4(xsrc, (uint32_t)((c * p.H + iy) * p.W + 4 * q) * 4u) : zero4;
                float* d = Xs + c * p.PLANE + r * p.PW + p.pw + 4 * q;
                d[0] = v.x; d[1] = v.y; d[2] = v.z; d[3] = v.w;
            }
        } else {
            for (int i = tid; i < BM * p.Kst; i += NT) {
                const int row = (int)p.div_kst.div((uint32_t)i), q = i - row * p.Kst;
                float v = 0.f;
                if (oc0 + row < p.Cout) v = gsrc[(i64)row * L + q];
                Gs[row * p.GP + q] = v;
            }
            for (int i = tid; i < CT * p.PR * p.W; i += NT) {
                const int c = (int)p.div_xcs.div((uint32_t)i), rem = i - c * (p.PR * p.W);
                const int r = (int)p.div_xrs.div((uint32_t)rem), q = rem - r * p.W;
                const int iy = iy0 + r;
                float v = 0.f;
                if (iy >= 0 && iy < p.H) v = xsrc[((i64)c * p.H + iy) * p.W + q];
                Xs[c * p.PLANE + r * p.PW + p.pw + q] = v;
            }
        }
    };

    const float* ga = Gs + (wave * 32 + l32) * p.GP + half;
    const float* xb = Xs + l32 * p.PLANE + half * p.sw;
    const int sw2 = 2 * p.sw;
    // One stage of MFMA work.  Two register sets alternate: while the MFMAs of one pixel pair run, the operands of
    // the next pair are read from LDS into the other set.  The reads past the end of a row land in the pitch
    // padding or in the slack behind the planes and are never used.
    auto compute = [&]() {
        for (int r = 0; r < p.R; ++r) {
            const float* gr = ga + r * p.ow;
            const float* x0 = xb + r * p.sh * p.PW;
            const float* x1 = x0 + p.PW;
            const float* x2 = x1 + p.PW;
            float a0, b0[KK], a1, b1[KK];
            auto rd = [&](float& a, float (&b)[KK], int j) {
                a = gr[j];
#pragma unroll
                for (int kx = 0; kx < KW; ++kx) { b[kx] = x0[kx]; b[KW + kx] = x1[kx]; b[2 * KW + kx] = x2[kx]; }
                x0 += sw2; x1 += sw2; x2 += sw2;
                __builtin_amdgcn_sched_barrier(0);
            };
            auto mma = [&](float a, const float (&b)[KK]) {
#pragma unroll
                for (int t = 0; t < KK; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b[t], acc[t], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            };
            rd(a0, b0, 0);
            int j = 0;
            for (; j + 4 <= p.ow; j += 4) {
                rd(a1, b1, j + 2);
                mma(a0, b0);
                rd(a0, b0, j + 4);
                mma(a1, b1);
            }
            if (j < p.ow) mma(a0, b0);
        }
    };

    const int s_beg = blockIdx.z * p.sps, s_end = min(p.stages, s_beg + p.sps);
    if constexpr (PREF) {
        if (s_beg < s_end) {
            prefetch(s_beg);
            park();
        }
        __syncthreads();
        for (int s = s_beg; s < s_end; ++s) {
            const bool more = s + 1 < s_end;
            if (more) prefetch(s + 1);
            // The other block on this CU may be staging: its address arithmetic must not win the issue slot over
            // this wave's MFMAs, so the MFMA loop runs at raised wave priority.
            __builtin_amdgcn_s_setprio(3);
            compute();
            __builtin_amdgcn_s_setprio(0);
            __syncthreads();
            if (more) park();
            __syncthreads();
        }
    } else {
        for (int s = s_beg; s < s_end; ++s) {
            stage_direct(s);
            __syncthreads();
            compute();
            __syncthreads();
        }
    }

    float* out = p.part + (i64)blockIdx.z * p.part_stride;
    const int ldo = KK * p.Cin;
#pragma unroll
    for (int t = 0; t < KK; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const int oc = oc0 + wave * 32 + igemm::Mfma<float>::row(e, lane);
            if (oc < p.Cout) out[(i64)oc * ldo + t * p.Cin + c0 + l32] = acc[t][e];
        }
}

// out[(oc*Cin + c)*KK + t] = sum_z part[z][oc][t][c], splits added in order.
__global__ __launch_bounds__(256) void wgrad_patch_reduce_kernel(const float* __restrict__ part, float* __restrict__ out, int n,
                                                                 int splits, int Cin, FastDiv div_row, FastDiv div_cin) {
    const int j = blockIdx.x * 256 + threadIdx.x;
    if (j >= n) return;
    float s = 0.f;
    int z = 0;
    for (; z + 8 <= splits; z += 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = part[(i64)(z + u) * n + j];
#pragma unroll
        for (int u = 0; u < 8; ++u) s = s + v[u];
    }
    for (; z < splits; ++z) s = s + part[(i64)z * n + j];
    const int oc = (int)div_row.div((uint32_t)j), rem = j - oc * (KK * Cin);
    const int t = (int)div_cin.div((uint32_t)rem), c = rem - t * Cin;
    out[((i64)oc * Cin + c) * KK + t] = s;
}

struct Plan {
    bool ok = false;
    int WM = 4, R = 1, PR = 0, PW = 0, PLANE = 0, GP = 0, Kst = 0, splits = 1, sps = 1, stages = 0;
    size_t smem = 0;
};

inline int odd_pitch(int n) { return (n + 30) / 32 * 32 + 1; }  // smallest pitch >= n with pitch % 32 == 1
inline int g_pitch(int n) { return odd_pitch(n); }    // smallest pitch >= n with pitch % 32 == 4

inline Plan make_plan(int num_cus, i64 B, i64 Cin, i64 H, i64 W, i64 Cout, i64 kh, i64 kw, i64 sh, i64 sw, i64 ph, i64 pw, i64 oh, i64 ow) {
    Plan pl;
    if (kh != KH || kw != KW || Cin % CT != 0 || ow % 2 != 0 || Cout < 32) return pl;
    if (W + 2 * pw > 4096 || sh > 8 || sw > 8) return pl;
    pl.WM = Cout > 64 ? 4 : 2;
    const int BM = 32 * pl.WM;
    int best = 0;
    for (int R = 1; R <= oh; ++R) {
        if (oh % R) continue;
        const int PR = (int)((R - 1) * sh + kh), PW = (int)(W + 2 * pw);
        const size_t smem = ((size_t)BM * g_pitch((int)(R * ow)) + (size_t)CT * odd_pitch(PR * PW) + SLACK) * sizeof(float);
        if (smem > LDS_BUDGET) break;
        best = R;
        if (R * ow >= 48) break;
    }
    if (!best) return pl;
    pl.R = best;
    pl.PR = (int)((best - 1) * sh + kh);
    pl.PW = (int)(W + 2 * pw);
    pl.PLANE = odd_pitch(pl.PR * pl.PW);
    pl.Kst = (int)(best * ow);
    pl.GP = g_pitch(pl.Kst);
    pl.smem = ((size_t)BM * pl.GP + (size_t)CT * pl.PLANE + SLACK) * sizeof(float);
    // the last tap of the last pixel of a stage must stay inside the plane
    if ((pl.PR - 1) * pl.PW + (ow - 1) * sw + kw - 1 >= pl.PLANE) return pl;
    pl.stages = (int)(B * (oh / best));
    const i64 tiles = (Cin / CT) * fx::ceil_div(Cout, (i64)BM);
    const i64 want = (i64)num_cus * 2;
    i64 splits = std::max<i64>(1, std::min<i64>(want / tiles, pl.stages));
    pl.sps = (int)fx::ceil_div((i64)pl.stages, splits);
    pl.splits = (int)fx::ceil_div((i64)pl.stages, (i64)pl.sps);
    if (pl.splits > 65535 || tiles > 65535 || Cout * Cin * KK > 0x7fffffff) return pl;
    pl.ok = true;
    return pl;
}

inline i64 workspace_bytes(const Plan& pl, i64 Cout, i64 Cin) { return (i64)pl.splits * Cout * Cin * KK * (i64)sizeof(float); }

inline int run(fx_ctx* c, const Plan& pl, const float* x, const float* g, float* dw, float* part, i64 Cin, i64 H, i64 W, i64 Cout,
               i64 sh, i64 sw, i64 ph, i64 pw, i64 oh, i64 ow) {
    Params p;
    p.x = x; p.g = g; p.part = part;
    p.Cin = (int)Cin; p.H = (int)H; p.W = (int)W; p.Cout = (int)Cout; p.oh = (int)oh; p.ow = (int)ow;
    p.sh = (int)sh; p.sw = (int)sw; p.ph = (int)ph; p.pw = (int)pw;
    p.R = pl.R; p.PR = pl.PR; p.PW = pl.PW; p.PLANE = pl.PLANE; p.GP = pl.GP; p.Kst = pl.Kst;
    p.stages = pl.stages; p.sps = pl.sps; p.spi = (int)(oh / pl.R);
    p.div_spi = FastDiv((uint32_t)p.spi);
    const bool vec = pl.Kst % 4 == 0 && W % 4 == 0 && ((uintptr_t)x % 16 == 0) && ((uintptr_t)g % 16 == 0);
    p.div_g4 = FastDiv((uint32_t)std::max(1, pl.Kst / 4));
    p.div_xc = FastDiv((uint32_t)std::max<i64>(1, pl.PR * (W / 4)));
    p.div_xr = FastDiv((uint32_t)std::max<i64>(1, W / 4));
    p.div_kst = FastDiv((uint32_t)pl.Kst);
    p.div_xcs = FastDiv((uint32_t)(pl.PR * W));
    p.div_xrs = FastDiv((uint32_t)W);
    p.part_stride = Cout * Cin * KK;
    const int BM = 32 * pl.WM;
    const dim3 grid((unsigned)(Cin / CT), (unsigned)fx::ceil_div(Cout, (i64)BM), (unsigned)pl.splits);
#define FX_WGP_LAUNCH(WMV, VECV, XRV)                                                                                 \
    do {                                                                                                              \
        static const hipError_t attr = hipFuncSetAttribute((const void*)wgrad_patch_kernel<WMV, VECV, XRV>,           \
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_BUDGET); \
        FX_HIP_CHECK(attr);                                                                                           \
        wgrad_patch_kernel<WMV, VECV, XRV><<<grid, dim3(64 * WMV), pl.smem, c->stream>>>(p);                          \
    } while (0)
    const bool pref = vec && pl.WM == 4 && pl.Kst <= 4 * LPR && W <= 4 * LPR;
    if (pref && pl.PR == 3) FX_WGP_LAUNCH(4, true, 3);
    else if (pref && pl.PR == 4) FX_WGP_LAUNCH(4, true, 4);
    else if (pl.WM == 4 && vec) FX_WGP_LAUNCH(4, true, 0);
    else if (pl.WM == 4) FX_WGP_LAUNCH(4, false, 0);
    else if (vec) FX_WGP_LAUNCH(2, true, 0);
    else FX_WGP_LAUNCH(2, false, 0);
#undef FX_WGP_LAUNCH
    FX_LAUNCH_CHECK();
    const int n = (int)p.part_stride;
    wgrad_patch_reduce_kernel<<<dim3((unsigned)fx::ceil_div((i64)n, 256)), dim3(256), 0, c->stream>>>(
        part, dw, n, pl.splits, (int)Cin, FastDiv((uint32_t)(KK * Cin)), FastDiv((uint32_t)Cin));
    FX_LAUNCH_CHECK();
    return FX_OK;
}

}  // namespace wgp
