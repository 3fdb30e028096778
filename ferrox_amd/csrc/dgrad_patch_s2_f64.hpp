// Data gradient of a 3x3 convolution of stride 2 and padding 1 over an even-sized map (f64), the twin of dgrad_patch_s2.hpp on
// v_mfma_f64_16x16x4_f64:
//   dx[b][c][iy][ix] = sum over (oc, ky, kx) with iy + 1 - ky = 2 oy, ix + 1 - kx = 2 ox of g[b][oc][oy][ox] * w[oc][c][ky][kx]
// (col2im(W2d^T . grad_out) in the reference, src/backend/storage/extensions/convolutions.rs:268-294).
//
// The input pixels of grid cell (i, j) -- (2i + py, 2j + px) -- receive only the taps of their parity class, all from the four
// grad_out pixels (i, j), (i, j+1), (i+1, j), (i+1, j+1):
//   (0,0): w11 g(i,j)                 (0,1): w10 g(i,j+1) + w12 g(i,j)                 (1,0): w01 g(i+1,j) + w21 g(i,j)
//   (1,1): w00 g(i+1,j+1) + w02 g(i+1,j) + w20 g(i,j+1) + w22 g(i,j)
// A block (8 waves) takes 256 cells of one image -- TR = 256 / OW grid rows -- and 32 input channels; a wave owns 32 cells and
// keeps, per class, 2 x 2 accumulator blocks of 16 (c) x 16 (cells).  The output channels are reduced in chunks of OCC, four
// per MFMA step; per chunk the block holds in LDS
//   Ws[oc quad][tap][c half][lane]   the MFMA A operand as the lanes read it: lane l holds w[oc = 4 quad + l / 16][c = 16 half + l % 16][tap]
//   Gs[oc][row][col]                 the (TR + 1) x (OW + 1) patch of grad_out (row TR is the next tile's first row or zero,
//                                    column OW is zero), odd plane pitch
// in two buffers: the next chunk is loaded into registers before the MFMA loop of the current one and parked after it, a chunk
// costs one barrier.  Per oc quad a wave reads 18 weights and 8 patch values for 36 MFMAs; the two waves of a SIMD cover each
// other's reads.  The two column classes of a cell are stored together as one 16-byte pair.
#pragma once
#include <cstdlib>

#include "igemm_core.hpp"

namespace dgd2 {
using igemm::FastDiv;
using igemm::f64x4;

constexpr int KK = 9, NT = 512, CT = 32, CELLS = 256;
constexpr size_t LDS_LIMIT = 160 * 1024;

struct Params {
    const double* g;
    const double* act;  // MASK: the ReLU output of the layer whose gradient g is; g is staged as g * (act > 0)
    const double* w;
    double* dx;
    int Cin, Cout, oh, tpi, nct;  // tiles per image, channel tiles
    FastDiv div_nct, div_tpi;
};

__device__ __forceinline__ double2 ldg2(const double* base, uint32_t byteoff) {
    typedef __attribute__((address_space(1))) const char gchar;
    typedef double v2 __attribute__((ext_vector_type(2)));
    typedef __attribute__((address_space(1))) const v2 gv2;
    const v2 v = *(gv2*)((gchar*)base + byteoff);
    return make_double2(v.x, v.y);
}

template <int OW, int OCC>
struct Shape {
    static constexpr int TR = CELLS / OW, PC = OW + 1, PR = TR + 1;
    static constexpr int GPL = (PR * PC) | 1;              // plane pitch of the patch
    static constexpr int KS = OCC / 4;                     // MFMA steps (oc quads) per chunk
    static constexpr int WCH = KS * KK * 2 * 64, GCH = OCC * GPL, BUF = WCH + GCH;
    static constexpr size_t LDS = 2 * (size_t)BUF * sizeof(double);
    static constexpr int W2 = OCC * CT * KK / 2;           // double2 of a weight chunk (32 x 9 contiguous doubles per oc)
    static constexpr int NWP = (W2 + NT - 1) / NT;         // passes over them
    static constexpr int NGP = OCC * (CELLS / 2) / NT;     // passes over the TR full rows of the patch (128 double2 per oc)
    static constexpr int X2 = OCC * OW / 2;                // double2 of the extra row
    static_assert(CELLS % OW == 0 && OW % 16 == 0 && OCC % 4 == 0 && OCC * (CELLS / 2) % NT == 0 && X2 <= NT && LDS <= LDS_LIMIT, "shape");
};

// MASK: grad_out arrives unmasked and the layer's ReLU is applied to the staged patch (g * (act > 0), the bits of fx_relu_bwd).
template <int OW, int OCC, bool MASK>
__global__ __launch_bounds__(NT, 1) void dgrad_s2_f64_kernel(const Params p) {
    using S = Shape<OW, OCC>;
    constexpr int TR = S::TR, PC = S::PC, GPL = S::GPL, KS = S::KS, WCH = S::WCH, BUF = S::BUF;
    FX_DYNAMIC_SMEM(double, smem_d);
    double* smem = smem_d;
    const int tid = threadIdx.x, lane = tid & 63, kq = lane >> 4, l16 = lane & 15;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int bt = (int)p.div_nct.div(blockIdx.x), ct = (int)blockIdx.x - bt * p.nct;
    const int b = (int)p.div_tpi.div((uint32_t)bt), tile = bt - b * p.tpi;
    const int c0 = ct * CT, i0 = tile * TR;
    const int L = p.oh * OW, H = 2 * p.oh, W = 2 * OW;
    const bool next_row = i0 + TR < p.oh;  // the patch's last row exists in grad_out (block-uniform)

    // staging maps (constant over the chunks)
    const double2 zero2 = make_double2(0., 0.);
    double2 wv[S::NWP], gv[S::NGP], xv, av[MASK ? S::NGP : 1], axv;
    const double* wsrc = p.w + (i64)c0 * KK;
    const double* gsrc = p.g + ((i64)b * p.Cout * p.oh + i0) * OW;
    const double* asrc = MASK ? p.act + ((i64)b * p.Cout * p.oh + i0) * OW : nullptr;
    auto masked = [](double2 v, const double2& a) __attribute__((always_inline)) {
        v.x = v.x * (a.x > 0. ? 1. : 0.);
        v.y = v.y * (a.y > 0. ? 1. : 0.);
        return v;
    };
    const int gq = tid & 127, goc = tid >> 7;                   // double2 of the tile's TR * OW doubles, oc within a pass of 4
    const int g_dst = goc * GPL + (gq / (OW / 2)) * PC + (gq % (OW / 2)) * 2;
    const uint32_t g_off = (uint32_t)(goc * L + 2 * gq) * 8u;
    const int xoc = tid / (OW / 2), xq = tid % (OW / 2);        // extra row: oc, double2 column
    const bool x_lane = tid < S::X2;
    const uint32_t x_off = x_lane ? (uint32_t)(xoc * L + TR * OW + 2 * xq) * 8u : 0u;
    auto prefetch = [&](int k) __attribute__((always_inline)) {
        const int oc0 = k * OCC;
#pragma unroll
        for (int u = 0; u < S::NWP; ++u) {
            const int f = u * NT + tid;
            const bool ok = (u + 1) * NT <= S::W2 || f < S::W2;
            const int ocl = f / 144, q = f - ocl * 144;
            wv[u] = ldg2(wsrc + (i64)oc0 * p.Cin * KK, ok ? (uint32_t)(ocl * p.Cin * KK + 2 * q) * 8u : 0u);
        }
#pragma unroll
        for (int u = 0; u < S::NGP; ++u) gv[u] = ldg2(gsrc + (i64)(oc0 + 4 * u) * L, g_off);
        if (next_row) xv = ldg2(gsrc + (i64)oc0 * L, x_off);
        else xv = zero2;
        if constexpr (MASK) {
#pragma unroll
            for (int u = 0; u < S::NGP; ++u) av[u] = ldg2(asrc + (i64)(oc0 + 4 * u) * L, g_off);
            if (next_row) axv = ldg2(asrc + (i64)oc0 * L, x_off);
            else axv = zero2;
        }
    };
    auto park = [&](int buf) __attribute__((always_inline)) {
        double* Ws = smem + buf * BUF;
        double* Gs = Ws + WCH;
#pragma unroll
        for (int u = 0; u < S::NWP; ++u) {
            const int f = u * NT + tid;
            if ((u + 1) * NT <= S::W2 || f < S::W2) {
                const int ocl = f / 144, q = f - ocl * 144;
                const double v[2] = {wv[u].x, wv[u].y};
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    const int e = 2 * q + i, c = e / KK, t = e - c * KK;
                    Ws[(((ocl >> 2) * KK + t) * 2 + (c >> 4)) * 64 + (ocl & 3) * 16 + (c & 15)] = v[i];
                }
            }
        }
#pragma unroll
        for (int u = 0; u < S::NGP; ++u) {
            double* d = Gs + g_dst + 4 * u * GPL;
            if constexpr (MASK) gv[u] = masked(gv[u], av[u]);
            d[0] = gv[u].x; d[1] = gv[u].y;
        }
        if (x_lane) {
            double* d = Gs + xoc * GPL + TR * PC + 2 * xq;
            if constexpr (MASK) xv = masked(xv, axv);
            d[0] = xv.x; d[1] = xv.y;
        }
    };

    f64x4 acc[2][2][2][2];  // [py][px][c half][cell half]
#pragma unroll
    for (int i = 0; i < 16; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[i >> 3][(i >> 2) & 1][(i >> 1) & 1][i & 1][e] = 0.;

    // this wave's cells: wave * 32 + 16 h + l16 of the tile (h = cell half), row-major; lane l reads the patch plane of
    // oc = 4 quad + l / 16
    int crow[2], ccol[2], gb0[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int cell = wave * 32 + 16 * h + l16;
        crow[h] = cell / OW;
        ccol[h] = cell % OW;
        gb0[h] = WCH + kq * GPL + crow[h] * PC + ccol[h];
    }
    auto compute = [&](int buf) __attribute__((always_inline)) {
        const double* wa = smem + buf * BUF + lane;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            double a[KK][2], bq[2][4];
#pragma unroll
            for (int t = 0; t < KK; ++t)
#pragma unroll
                for (int ch = 0; ch < 2; ++ch) a[t][ch] = wa[((ks * KK + t) * 2 + ch) * 64];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const double* gb = smem + buf * BUF + gb0[h] + 4 * ks * GPL;
                bq[h][0] = gb[0];
                bq[h][1] = gb[1];
                bq[h][2] = gb[PC];
                bq[h][3] = gb[PC + 1];
            }
            __builtin_amdgcn_sched_barrier(0);
            // taps w[ky][kx] = a[3 ky + kx]; b: 0 = g(i,j), 1 = g(i,j+1), 2 = g(i+1,j), 3 = g(i+1,j+1).  Tap by tap over the four
            // (c half, cell half) blocks: no MFMA waits for the one before it.
#define FX_DGD2_STEP(PY, PX, T, BI)                                                                                          \
    _Pragma("unroll") for (int ch = 0; ch < 2; ++ch) _Pragma("unroll") for (int h = 0; h < 2; ++h)                            \
        acc[PY][PX][ch][h] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[T][ch], bq[h][BI], acc[PY][PX][ch][h], 0, 0, 0);
            FX_DGD2_STEP(1, 1, 0, 3)
            FX_DGD2_STEP(0, 0, 4, 0)
            FX_DGD2_STEP(1, 1, 2, 2)
            FX_DGD2_STEP(0, 1, 3, 1)
            FX_DGD2_STEP(1, 1, 6, 1)
            FX_DGD2_STEP(1, 0, 1, 2)
            FX_DGD2_STEP(1, 1, 8, 0)
            FX_DGD2_STEP(0, 1, 5, 0)
            FX_DGD2_STEP(1, 0, 7, 0)
#undef FX_DGD2_STEP
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    const int nchunks = p.Cout / OCC;
    prefetch(0);
    // column OW of every patch row is the zero padding right of the map: written once in both buffers
    for (int i = tid; i < 2 * OCC * S::PR; i += NT) {
        const int buf = i / (OCC * S::PR), rem = i - buf * (OCC * S::PR), oc = rem / S::PR, r = rem - oc * S::PR;
        smem[buf * BUF + WCH + oc * GPL + r * PC + OW] = 0.;
    }
    park(0);
    __syncthreads();
    int cur = 0;
    for (int k = 0; k < nchunks; ++k) {
        const bool more = k + 1 < nchunks;
        if (more) prefetch(k + 1);
        compute(cur);
        // the other buffer was last read in the chunk before this one, which every wave has left through the barrier below
        if (more) park(cur ^ 1);
        __syncthreads();
        cur ^= 1;
    }

    // dx[b][c][2 (i0 + crow) + py][2 ccol + px]: the two column classes of a cell as one pair
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        double* out = p.dx + (((i64)b * p.Cin + c0) * H + 2 * (i0 + crow[h])) * W + 2 * ccol[h];
#pragma unroll
        for (int ch = 0; ch < 2; ++ch)
#pragma unroll
            for (int py = 0; py < 2; ++py)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int c = 16 * ch + igemm::Mfma<double>::row(e, lane);
                    *reinterpret_cast<double2*>(out + ((i64)c * H + py) * W) = make_double2(acc[py][0][ch][h][e], acc[py][1][ch][h][e]);
                }
    }
}

struct Plan {
    bool ok = false;
    int OW = 0, OCC = 0;
    size_t smem = 0;
};

// Instantiated (OW, OCC): maps 32 and 64 wide.  Chunks of 16 output channels measured level with chunks of 8 (55.2 against
// 55.3 us at [256,32,32,32] <- 64) at twice the LDS.
#define FX_DGD2_SHAPES(X) X(16, 8) X(32, 8)

inline Plan make_plan(i64 B, i64 Cin, i64 H, i64 W, i64 Cout, i64 kh, i64 kw, i64 sh, i64 sw, i64 ph, i64 pw, i64 oh, i64 ow) {
    Plan pl;
    if (kh != 3 || kw != 3 || sh != 2 || sw != 2 || ph != 1 || pw != 1 || W != 2 * ow || H != 2 * oh || Cin % CT != 0) return pl;
    if (Cout * oh * ow * 8 > 0x7fffffff || Cout * Cin * KK * 8 > 0x7fffffff || B * (Cin / CT) * oh > 0x7fffffff) return pl;
#define FX_DGD2_PICK(O, C_)                                                                  \
    if (!pl.ok && ow == O && Cout % C_ == 0 && oh % (CELLS / O) == 0) {                      \
        pl.ok = true; pl.OW = O; pl.OCC = C_; pl.smem = Shape<O, C_>::LDS;                   \
    }
    FX_DGD2_SHAPES(FX_DGD2_PICK)
#undef FX_DGD2_PICK
    return pl;
}

// g, w and dx must be 16-byte aligned.
// act non-null: the masked variant (act 16-byte aligned as well).
inline int run(fx_ctx* c, const Plan& pl, const double* g, const double* w, double* dx, i64 B, i64 Cin, i64 Cout, i64 oh,
               const double* act = nullptr) {
    Params p;
    p.g = g; p.w = w; p.dx = dx; p.act = act;
    p.Cin = (int)Cin; p.Cout = (int)Cout; p.oh = (int)oh;
    p.tpi = (int)(oh / (CELLS / pl.OW));
    p.nct = (int)(Cin / CT);
    p.div_nct = FastDiv((uint32_t)p.nct);
    p.div_tpi = FastDiv((uint32_t)p.tpi);
    const dim3 grid((unsigned)(B * p.tpi * p.nct));
    bool launched = false;
#define FX_DGD2_LAUNCH(O, C_)                                                                                          \
    if (!launched && pl.OW == O && pl.OCC == C_) {                                                                     \
        static const hipError_t attr = hipFuncSetAttribute((const void*)dgrad_s2_f64_kernel<O, C_, false>,             \
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_LIMIT); \
        static const hipError_t attr_m = hipFuncSetAttribute((const void*)dgrad_s2_f64_kernel<O, C_, true>,            \
                                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_LIMIT); \
        FX_HIP_CHECK(attr);                                                                                            \
        FX_HIP_CHECK(attr_m);                                                                                          \
        if (act) FX_LAUNCH(grid, dim3(NT), pl.smem, c->stream, (p), dgrad_s2_f64_kernel<O, C_, true>);                          \
        else FX_LAUNCH(grid, dim3(NT), pl.smem, c->stream, (p), dgrad_s2_f64_kernel<O, C_, false>);                             \
        launched = true;                                                                                               \
    }
    FX_DGD2_SHAPES(FX_DGD2_LAUNCH)
#undef FX_DGD2_LAUNCH
    FX_REQUIRE(launched, "dgrad stride-2 patch kernel (f64): unexpected shape (%d, %d)", pl.OW, pl.OCC);
    FX_LAUNCH_CHECK();
    return FX_OK;
}

}  // namespace dgd2
