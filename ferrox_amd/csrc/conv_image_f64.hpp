// Forward pass of a 3x3 convolution of stride 1 and padding 1 over an image of 1 to 4 channels (f64) on
// v_mfma_f64_16x16x4_f64: the first layer of the reference's networks (examples/common/models.rs:200-318; the product is
// conv2d_impl, src/backend/storage/extensions/convolutions.rs:218-266) in the precision whose general path, the implicit GEMM,
// gathers a K x pixels operand of K = Cin * 9 <= 36 that is mostly the padding of its 16-deep slabs.
//   y[b][oc][oy][ox] = bias[oc] + sum over (c, ky, kx) of w[oc][c][ky][kx] * x[b][c][oy + ky - 1][ox + kx - 1]
//
// The channels are one MFMA step (4, the missing ones a zero plane), so a tile is 9 taps and nothing else: a block (8 waves)
// takes 256 output pixels of one image -- TR = 256 / W rows -- and 32 output channels, a wave 32 pixels x 32 channels as 2 x 2
// accumulator blocks of 16 x 16, 36 MFMAs in all.  In LDS
//   Ws[tap][oc block][lane]   the A operand as the lanes read it: lane l holds w[oc = 16 block + l % 16][c = l / 16][tap]
//   Xs[c][row][col]           the TR + 2 zero-padded patch rows of the 4 channel planes (odd plane pitch)
// One load, one barrier, 36 MFMAs, the stores: the kernel is bound by the 8 bytes per output it writes, and several blocks per
// CU overlap each other's phases.  Bias (+ReLU) ride in the store.
#pragma once
#include <cstdlib>

#include "igemm_core.hpp"

namespace cim {
using igemm::FastDiv;
using igemm::f64x4;

constexpr int KK = 9, NT = 512, PIX = 256, CP = 4;

struct Params {
    const double* x;
    const double* w;
    double* y;
    const double* bias;  // or null
    int relu;
    int Cin, Cout, H, tpi, nmt;  // tiles per image, tiles of 32 output channels
    FastDiv div_nmt, div_tpi;
};

template <int W>
struct Shape {
    static constexpr int TR = PIX / W, PR = TR + 2, PW = W + 2;
    static constexpr int PLANE = (PR * PW) | 1;
    static constexpr int WCH = KK * 2 * 64, XCH = CP * PLANE;
    static constexpr int X2 = CP * PR * (W / 2);  // double2 of the patch, all four planes
    static_assert(PIX % W == 0 && W % 16 == 0 && X2 <= 2 * NT, "shape");
};

template <int W, bool BIAS>
__global__ __launch_bounds__(NT) void image_fwd_f64_kernel(const Params p) {
    using S = Shape<W>;
    constexpr int TR = S::TR, PR = S::PR, PW = S::PW, PLANE = S::PLANE, WCH = S::WCH;
    __shared__ __align__(16) double smem[S::WCH + S::XCH];
    double* Ws = smem;
    double* Xs = smem + WCH;
    const int tid = threadIdx.x, lane = tid & 63, kq = lane >> 4, l16 = lane & 15;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int bt = (int)p.div_nmt.div(blockIdx.x), mt = (int)blockIdx.x - bt * p.nmt;
    const int b = (int)p.div_tpi.div((uint32_t)bt), tile = bt - b * p.tpi;
    const int oc0 = mt * 32, oy0 = tile * TR, iy0 = oy0 - 1;
    const int L = p.H * W, K = p.Cin * KK;

    // the bias of the rows this lane stores, loaded up front
    double bv[2][4];
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int e = 0; e < 4; ++e) bv[m][e] = BIAS ? p.bias[oc0 + 16 * m + igemm::Mfma<double>::row(e, lane)] : 0.;

    // weights: element i of the 32 x (4 x 9) image, zero for the channels past Cin (rows of K = Cin * 9 doubles in w: 8-byte loads)
    for (int i = tid; i < 32 * CP * KK; i += NT) {
        const int ocl = i / (CP * KK), r = i - ocl * (CP * KK), cl = r / KK, t = r - cl * KK;
        const double v = cl < p.Cin ? p.w[(i64)(oc0 + ocl) * K + cl * KK + t] : 0.;
        Ws[(t * 2 + (ocl >> 4)) * 64 + cl * 16 + (ocl & 15)] = v;
    }
    // patch: double2 f -> (plane, row, 2 columns); rows outside the image and planes past Cin are zero
    const double* xsrc = p.x + (i64)b * p.Cin * L;
#pragma unroll
    for (int u = 0; u < (S::X2 + NT - 1) / NT; ++u) {
        const int f = u * NT + tid;
        if (f < S::X2) {
            const int cr = f / (W / 2), q = f - cr * (W / 2), c = cr / PR, r = cr - c * PR;
            const int iy = iy0 + r;
            double2 v = make_double2(0., 0.);
            if (c < p.Cin && iy >= 0 && iy < p.H) v = *reinterpret_cast<const double2*>(xsrc + ((i64)c * p.H + iy) * W + 2 * q);
            double* d = Xs + c * PLANE + r * PW + 1 + 2 * q;
            d[0] = v.x;
            d[1] = v.y;
        }
    }
    // the zero columns left and right of the map
    for (int i = tid; i < CP * PR * 2; i += NT) {
        const int cr = i >> 1;
        Xs[(cr / PR) * PLANE + (cr % PR) * PW + (i & 1) * (W + 1)] = 0.;
    }
    __syncthreads();

    f64x4 acc[2][2];  // [block of 16 output channels][pixel half]
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[m][h][e] = 0.;
    int xb0[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int pix = wave * 32 + 16 * h + l16;
        xb0[h] = kq * PLANE + (pix / W) * PW + pix % W;
    }
    double a[KK][2], bq[KK][2];
#pragma unroll
    for (int t = 0; t < KK; ++t) {
        const int ky = t / 3, kx = t % 3;
#pragma unroll
        for (int m = 0; m < 2; ++m) a[t][m] = Ws[(t * 2 + m) * 64 + lane];
#pragma unroll
        for (int h = 0; h < 2; ++h) bq[t][h] = Xs[xb0[h] + ky * PW + kx];
    }
#pragma unroll
    for (int t = 0; t < KK; ++t)
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
            for (int h = 0; h < 2; ++h) acc[m][h] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[t][m], bq[t][h], acc[m][h], 0, 0, 0);

#pragma unroll
    for (int h = 0; h < 2; ++h) {
        double* out = p.y + ((i64)b * p.Cout + oc0) * L + (i64)oy0 * W + wave * 32 + 16 * h + l16;
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int oc = 16 * m + igemm::Mfma<double>::row(e, lane);
                double v = acc[m][h][e];
                if constexpr (BIAS) {
                    v = v + bv[m][e];
                    if (p.relu) v = v > 0. ? v : 0.;
                }
                out[(i64)oc * L] = v;
            }
    }
}

// Maps 32 wide (8 rows per tile), heights a multiple of 8, output channels a multiple of 32.
inline bool eligible(i64 B, i64 Cin, i64 H, i64 W, i64 Cout, i64 kh, i64 kw, i64 sh, i64 sw, i64 ph, i64 pw) {
    return kh == 3 && kw == 3 && sh == 1 && sw == 1 && ph == 1 && pw == 1 && Cin >= 1 && Cin <= CP && W == 32 && H % (PIX / 32) == 0 &&
           Cout % 32 == 0 && B * (H / (PIX / 32)) * (Cout / 32) <= 0x7fffffff;
}

// x and y must be 16-byte aligned.
inline int run(fx_ctx* c, const double* x, const double* w, double* y, i64 B, i64 Cin, i64 H, i64 Cout, const double* bias, int relu) {
    Params p;
    p.x = x; p.w = w; p.y = y; p.bias = bias; p.relu = relu;
    p.Cin = (int)Cin; p.Cout = (int)Cout; p.H = (int)H;
    p.tpi = (int)(H / (PIX / 32));
    p.nmt = (int)(Cout / 32);
    p.div_nmt = FastDiv((uint32_t)p.nmt);
    p.div_tpi = FastDiv((uint32_t)p.tpi);
    const dim3 grid((unsigned)(B * p.tpi * p.nmt));
    if (bias) FX_LAUNCH(grid, dim3(NT), 0, c->stream, (p), image_fwd_f64_kernel<32, true>);
    else FX_LAUNCH(grid, dim3(NT), 0, c->stream, (p), image_fwd_f64_kernel<32, false>);
    FX_LAUNCH_CHECK();
    return FX_OK;
}

// ---- weight gradient of the same layer (1 to 3 channels: K = Cin * 9 <= 27 <= 32) -------------------------------------------
//   dw[oc][c][ky][kx] = sum over (b, oy, ox) of g[b][oc][oy][ox] * x[b][c][oy + ky - 1][ox + kx - 1]
// (grad_out_2d . im2col(x)^T, convolutions.rs:296-338).  The MFMA's 16 columns are (channel, tap) pairs -- two blocks of 16 hold
// the K <= 27 of them -- its reduction runs over 4 pixels: lane l reads g[oc = l % 16 (+ 16)][pixel + l / 16] and
// x[c][pixel + l / 16 shifted by the tap] for its pair (c, tap) = 16 block + l % 16, both from LDS, where a block has staged
// 32 rows of g (256 pixels of one image, odd pitch) and the padded patch under them.  A wave takes one row of 32 pixels: 8 steps
// of 4 MFMAs.  A block walks its range of tiles with the sums in registers, adds its eight waves' sums through LDS in wave
// order and leaves one partial sum, laid out like dw; the ordered split sum adds the partials.  Bound by the one read of g.
struct WParams {
    const double* x;
    const double* g;
    const double* act;  // MASK: the layer's ReLU output; g is staged as g * (act > 0)
    double* part;       // [splits][Cout][Cin * 9] (MASK: + [Cout] sums of the masked g behind each: the bias gradient)
    i64 part_stride;    // doubles between the partial sums of two splits
    int Cin, Cout, H, tpi;
    int tiles, tps;  // B * tiles per image, tiles per split
    FastDiv div_tpi;
};

constexpr int GPITCH = PIX + 1;

// MASK: the gradient arrives unmasked and this layer's ReLU is applied while g is staged (g * (act > 0), the bits of
// fx_relu_bwd); pair index K <= 27 of the 32 is free, and with an operand of 1.0 there the MFMA leaves the sums of the masked g
// over the pixels in it: the bias gradient.
template <bool MASK>
__global__ __launch_bounds__(NT) void image_wgrad_f64_kernel(const WParams p) {
    using S = Shape<32>;
    constexpr int W = 32, TR = S::TR, PR = S::PR, PW = S::PW, PLANE = S::PLANE;
    FX_DYNAMIC_SMEM(double, smem_w);
    double* Gs = smem_w;                   // [32 oc][GPITCH]
    double* Xs = smem_w + 32 * GPITCH;     // [CP planes][PR][PW], odd plane pitch
    const int tid = threadIdx.x, lane = tid & 63, kq = lane >> 4, l16 = lane & 15;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int oc0 = blockIdx.y * 32, L = p.H * W, K = p.Cin * KK;
    const int t_beg = blockIdx.x * p.tps, t_end = min(p.tiles, t_beg + p.tps);

    // this lane's (channel, tap) pairs: 16 nb + l16; pairs past K read a valid address and contribute zeros
    int xoff[2];
    bool pair_ok[2], pair_one[2];
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
        const int kp = 16 * nb + l16;
        pair_ok[nb] = kp < K;
        pair_one[nb] = MASK && kp == K;
        const int c = pair_ok[nb] ? kp / KK : 0, t = pair_ok[nb] ? kp % KK : 0;
        xoff[nb] = c * PLANE + (wave + t / 3) * PW + t % 3 + kq;  // pixel (row wave, column 4 s + kq): + 4 s per step
    }
    const int goff = l16 * GPITCH + wave * W + kq;                // + 16 GPITCH for the second block of output channels

    f64x4 acc[2][2];  // [oc block][pair block]
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[m][nb][e] = 0.;
    // the zero columns left and right of the map stay zero over the tiles
    for (int i = tid; i < CP * PR * 2; i += NT) {
        const int cr = i >> 1;
        Xs[(cr / PR) * PLANE + (cr % PR) * PW + (i & 1) * (W + 1)] = 0.;
    }
    for (int tl = t_beg; tl < t_end; ++tl) {
        const int b = (int)p.div_tpi.div((uint32_t)tl), tile = tl - b * p.tpi;
        const int oy0 = tile * TR, iy0 = oy0 - 1;
        // g: 32 rows of 256 doubles, 8 double2 per thread
        const double* gsrc = p.g + ((i64)b * p.Cout + oc0) * L + (i64)oy0 * W;
        double2 gv[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int f = u * NT + tid, row = f >> 7, q = f & 127;
            gv[u] = *reinterpret_cast<const double2*>(gsrc + (i64)row * L + 2 * q);
            if constexpr (MASK) {
                const double2 a = *reinterpret_cast<const double2*>(p.act + (gsrc - p.g) + (i64)row * L + 2 * q);
                gv[u].x = gv[u].x * (a.x > 0. ? 1. : 0.);
                gv[u].y = gv[u].y * (a.y > 0. ? 1. : 0.);
            }
        }
        const double* xsrc = p.x + (i64)b * p.Cin * L;
        double2 xv[2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int f = u * NT + tid;
            xv[u] = make_double2(0., 0.);
            if (f < S::X2) {
                const int cr = f / (W / 2), q = f - cr * (W / 2), c = cr / PR, r = cr - c * PR;
                const int iy = iy0 + r;
                if (c < p.Cin && iy >= 0 && iy < p.H) xv[u] = *reinterpret_cast<const double2*>(xsrc + ((i64)c * p.H + iy) * W + 2 * q);
            }
        }
        __syncthreads();  // the tile before has been read
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int f = u * NT + tid, row = f >> 7, q = f & 127;
            double* d = Gs + row * GPITCH + 2 * q;
            d[0] = gv[u].x;
            d[1] = gv[u].y;
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int f = u * NT + tid;
            if (f < S::X2) {
                const int cr = f / (W / 2), q = f - cr * (W / 2), c = cr / PR, r = cr - c * PR;
                double* d = Xs + c * PLANE + r * PW + 1 + 2 * q;
                d[0] = xv[u].x;
                d[1] = xv[u].y;
            }
        }
        __syncthreads();
#pragma unroll
        for (int s = 0; s < W / 4; ++s) {
            const double a0 = Gs[goff + 4 * s], a1 = Gs[goff + 16 * GPITCH + 4 * s];
            double b0 = Xs[xoff[0] + 4 * s], b1 = Xs[xoff[1] + 4 * s];
            if (!pair_ok[0]) b0 = pair_one[0] ? 1. : 0.;
            if (!pair_ok[1]) b1 = pair_one[1] ? 1. : 0.;
            acc[0][0] = __builtin_amdgcn_mfma_f64_16x16x4f64(a0, b0, acc[0][0], 0, 0, 0);
            acc[0][1] = __builtin_amdgcn_mfma_f64_16x16x4f64(a0, b1, acc[0][1], 0, 0, 0);
            acc[1][0] = __builtin_amdgcn_mfma_f64_16x16x4f64(a1, b0, acc[1][0], 0, 0, 0);
            acc[1][1] = __builtin_amdgcn_mfma_f64_16x16x4f64(a1, b1, acc[1][1], 0, 0, 0);
        }
    }
    // the eight waves' sums through LDS (the stage buffers are free after a barrier), added in wave order by waves 0 .. 3
    __syncthreads();
    double* red = smem_w;  // [8 waves][16 elements][64 lanes]
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
#pragma unroll
            for (int e = 0; e < 4; ++e) red[(wave * 16 + 4 * (2 * m + nb) + e) * 64 + lane] = acc[m][nb][e];
    __syncthreads();
    double* out = p.part + (i64)blockIdx.x * p.part_stride + (i64)oc0 * K;
    double* bout = p.part + (i64)blockIdx.x * p.part_stride + (i64)p.Cout * K + oc0;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const int el = 2 * wave + u, blk = el >> 2, e = el & 3;  // wave w finishes elements 2 w and 2 w + 1
        double v = red[el * 64 + lane];
#pragma unroll
        for (int w = 1; w < 8; ++w) v = v + red[(w * 16 + el) * 64 + lane];
        const int oc = 16 * (blk >> 1) + 4 * e + kq, kp = 16 * (blk & 1) + l16;
        if (kp < K) out[(i64)oc * K + kp] = v;
        if (MASK && kp == K) bout[oc] = v;
    }
}

struct WPlan {
    bool ok = false;
    int splits = 1, tps = 1, tiles = 0;
};

inline WPlan wgrad_plan(int num_cus, i64 B, i64 Cin, i64 H, i64 W, i64 Cout, i64 kh, i64 kw, i64 sh, i64 sw, i64 ph, i64 pw) {
    WPlan pl;
    if (kh != 3 || kw != 3 || sh != 1 || sw != 1 || ph != 1 || pw != 1 || Cin < 1 || Cin > 3 || W != 32 || H % (PIX / 32) != 0 || Cout % 32 != 0)
        return pl;
    const i64 tiles = B * (H / (PIX / 32)), rows = Cout / 32;
    if (tiles > 0x7fffffff || rows > 65535) return pl;
    // two blocks per CU (78 KB of LDS each); at least two tiles per block where there are that many
    const i64 splits = std::max<i64>(1, std::min<i64>(2 * (i64)num_cus / rows, std::max<i64>(1, tiles / 2)));
    pl.tps = (int)fx::ceil_div(tiles, splits);
    pl.splits = (int)fx::ceil_div(tiles, (i64)pl.tps);
    pl.tiles = (int)tiles;
    pl.ok = true;
    return pl;
}
// the masked variant keeps [Cout] bias sums behind every split's partial
inline i64 wgrad_workspace_bytes(const WPlan& pl, i64 Cout, i64 Cin, bool with_bias = false) {
    return (i64)pl.splits * (Cout * Cin * KK + (with_bias ? Cout : 0)) * (i64)sizeof(double);
}

// x, g and part must be 16-byte aligned.
// act / db non-null: the masked variant (act 16-byte aligned as well).
inline int run_wgrad(fx_ctx* c, const WPlan& pl, const double* x, const double* g, double* dw, double* part, i64 Cin, i64 H, i64 Cout,
                     const double* act = nullptr, double* db = nullptr) {
    WParams p;
    p.x = x; p.g = g; p.part = part; p.act = act;
    p.part_stride = Cout * Cin * KK + (act ? Cout : 0);
    p.Cin = (int)Cin; p.Cout = (int)Cout; p.H = (int)H;
    p.tpi = (int)(H / (PIX / 32));
    p.tiles = pl.tiles; p.tps = pl.tps;
    p.div_tpi = FastDiv((uint32_t)p.tpi);
    const size_t lds = std::max((size_t)(32 * GPITCH + Shape<32>::XCH), (size_t)8 * 16 * 64) * sizeof(double);
    static const hipError_t attr = hipFuncSetAttribute((const void*)image_wgrad_f64_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024);
    static const hipError_t attr_m = hipFuncSetAttribute((const void*)image_wgrad_f64_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024);
    FX_HIP_CHECK(attr);
    FX_HIP_CHECK(attr_m);
    const dim3 grid((unsigned)pl.splits, (unsigned)(Cout / 32));
    if (act) FX_LAUNCH(grid, dim3(NT), lds, c->stream, (p), image_wgrad_f64_kernel<true>);
    else FX_LAUNCH(grid, dim3(NT), lds, c->stream, (p), image_wgrad_f64_kernel<false>);
    FX_LAUNCH_CHECK();
    if (act) return igemm::launch_splitk_reduce_pair<double>(c, part, p.part_stride, pl.splits, dw, Cout * Cin * KK, db, Cout);
    return igemm::launch_splitk_reduce<double>(c, part, dw, Cout * Cin * KK, pl.splits);
}

}  // namespace cim
