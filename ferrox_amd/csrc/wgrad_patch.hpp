// Weight gradient of a 3x3 convolution (f32) with both operands staged in LDS in their natural layouts.
//
// dw[oc][c][ky][kx] = sum over (b, oy, ox) of g[b][oc][oy][ox] * x[b][c][oy*sh+ky-ph][ox*sw+kx-pw]
// (the product the reference forms as grad_out_2d . im2col(x)^T, src/backend/storage/extensions/convolutions.rs:296-338).
//
// One stage = R output rows of one image.  A block copies, per stage,
//   Gs[oc][pixel]      BM output-channel rows of g, pixels contiguous as in memory  (pitch GP,    GP % 32 == 1)
//   Xs[c][row][col]    32 input-channel planes of the zero-padded rows those pixels touch (pitch PLANE % 32 == 1)
// and every wave then runs 9 accumulator blocks of 32(oc) x 32(c), one per filter tap: the MFMA A operand of lane l
// is Gs[oc = l%32][pixel + l/32], the B operand of tap (ky,kx) is Xs[c = l%32][that pixel shifted by (ky,kx)].
// The odd pitches put the 32 lanes of a half-wave on 32 different LDS banks for both reads.  The patch is
// loaded once and serves all nine taps, so no im2col gather or bounds test is left in the MFMA loop.
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


// PREF: the next stage's global loads are issued before the MFMA loop of the current stage and parked in
// registers, NG float4 of g and NX float4 of x per thread (needs VEC); otherwise a stage is loaded, then used.
template <int WM, bool VEC, int NG, int NX>
__global__ __launch_bounds__(64 * WM, 2) void wgrad_patch_kernel(const Params p) {
    constexpr bool PREF = NG > 0;
    static_assert(VEC || !PREF, "prefetch needs the vector path");
    constexpr int NT = 64 * WM, BM = 32 * WM;
    extern __shared__ float smem[];
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

    float4 gv[PREF ? NG : 1], xv[PREF ? NX : 1];
    const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);

    auto stage_ptrs = [&](int s, const float*& gsrc, const float*& xsrc, int& iy0) {
        const int b = (int)p.div_spi.div((uint32_t)s);
        const int oy0 = (s - b * p.spi) * p.R;
        iy0 = oy0 * p.sh - p.ph;
        gsrc = p.g + ((i64)b * p.Cout + oc0) * L + (i64)oy0 * p.ow;
        xsrc = p.x + ((i64)b * p.Cin + c0) * p.H * p.W;
    };
    auto g_load4 = [&](const float* gsrc, int i) {
        const int row = (int)p.div_g4.div((uint32_t)i), q = i - row * k4;
        return (i < ng4 && oc0 + row < p.Cout) ? *reinterpret_cast<const float4*>(gsrc + (i64)row * L + 4 * q) : zero4;
    };
    auto g_store4 = [&](int i, const float4& v) {
        if (i < ng4) {
            const int row = (int)p.div_g4.div((uint32_t)i), q = i - row * k4;
            float* d = Gs + row * p.GP + 4 * q;
            d[0] = v.x; d[1] = v.y; d[2] = v.z; d[3] = v.w;
        }
    };
    auto x_load4 = [&](const float* xsrc, int iy0, int i) {
        const int c = (int)p.div_xc.div((uint32_t)i), rem = i - c * (p.PR * w4);
        const int r = (int)p.div_xr.div((uint32_t)rem), q = rem - r * w4;
        const int iy = iy0 + r;
        return (i < nx4 && iy >= 0 && iy < p.H) ? *reinterpret_cast<const float4*>(xsrc + ((i64)c * p.H + iy) * p.W + 4 * q) : zero4;
    };
    auto x_store4 = [&](int i, const float4& v) {
        if (i < nx4) {
            const int c = (int)p.div_xc.div((uint32_t)i), rem = i - c * (p.PR * w4);
            const int r = (int)p.div_xr.div((uint32_t)rem), q = rem - r * w4;
            float* d = Xs + c * p.PLANE + r * p.PW + p.pw + 4 * q;
            d[0] = v.x; d[1] = v.y; d[2] = v.z; d[3] = v.w;
        }
    };
    auto prefetch = [&](int s) {
        const float *gsrc, *xsrc;
        int iy0, t0 = tid;
        asm volatile("" : "+v"(t0));  // keeps the per-stage index arithmetic out of long-lived registers
        stage_ptrs(s, gsrc, xsrc, iy0);
#pragma unroll
        for (int u = 0; u < NG; ++u) gv[PREF ? u : 0] = g_load4(gsrc, t0 + u * NT);
#pragma unroll
        for (int u = 0; u < NX; ++u) xv[PREF ? u : 0] = x_load4(xsrc, iy0, t0 + u * NT);
    };
    auto park = [&]() {
        int t0 = tid;
        asm volatile("" : "+v"(t0));
#pragma unroll
        for (int u = 0; u < NG; ++u) g_store4(t0 + u * NT, gv[PREF ? u : 0]);
#pragma unroll
        for (int u = 0; u < NX; ++u) x_store4(t0 + u * NT, xv[PREF ? u : 0]);
    };
    auto stage_direct = [&](int s) {
        const float *gsrc, *xsrc;
        int iy0;
        stage_ptrs(s, gsrc, xsrc, iy0);
        if constexpr (VEC) {
            for (int i = tid; i < ng4; i += NT) g_store4(i, g_load4(gsrc, i));
            for (int i = tid; i < nx4; i += NT) x_store4(i, x_load4(xsrc, iy0, i));
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
            compute();
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
        const size_t smem = ((size_t)BM * odd_pitch((int)(R * ow)) + (size_t)CT * odd_pitch(PR * PW) + SLACK) * sizeof(float);
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
    pl.GP = odd_pitch(pl.Kst);
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
#define FX_WGP_LAUNCH(WMV, VECV, NGV, NXV)                                                                            \
    do {                                                                                                              \
        static const hipError_t attr = hipFuncSetAttribute((const void*)wgrad_patch_kernel<WMV, VECV, NGV, NXV>,      \
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_BUDGET); \
        FX_HIP_CHECK(attr);                                                                                           \
        wgrad_patch_kernel<WMV, VECV, NGV, NXV><<<grid, dim3(64 * WMV), pl.smem, c->stream>>>(p);                     \
    } while (0)
#define FX_WGP_DISPATCH(WMV)                                                                                          \
    do {                                                                                                              \
        if (vec && ng <= 4 && nx <= 4) FX_WGP_LAUNCH(WMV, true, 4, 4);                                                \
        else if (vec && ng <= 7 && nx <= 6) FX_WGP_LAUNCH(WMV, true, 7, 6);                                           \
        else if (vec) FX_WGP_LAUNCH(WMV, true, 0, 0);                                                                 \
        else FX_WGP_LAUNCH(WMV, false, 0, 0);                                                                         \
    } while (0)
    const int NT = 64 * pl.WM;  // float4 loads per thread and stage: ng of g, nx of x
    const i64 ng = fx::ceil_div((i64)BM * (pl.Kst / 4), (i64)NT), nx = fx::ceil_div((i64)CT * pl.PR * (W / 4), (i64)NT);
    if (pl.WM == 4) FX_WGP_DISPATCH(4);
    else FX_WGP_DISPATCH(2);
#undef FX_WGP_DISPATCH
#undef FX_WGP_LAUNCH
    FX_LAUNCH_CHECK();
    const int n = (int)p.part_stride;
    wgrad_patch_reduce_kernel<<<dim3((unsigned)fx::ceil_div((i64)n, 256)), dim3(256), 0, c->stream>>>(
        part, dw, n, pl.splits, (int)Cin, FastDiv((uint32_t)(KK * Cin)), FastDiv((uint32_t)Cin));
    FX_LAUNCH_CHECK();
    return FX_OK;
}

}  // namespace wgp
