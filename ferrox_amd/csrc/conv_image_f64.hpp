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
    static const bool off = [] { const char* v = getenv("FX_CIM"); return v && atoi(v) == 0; }();
    return !off && kh == 3 && kw == 3 && sh == 1 && sw == 1 && ph == 1 && pw == 1 && Cin >= 1 && Cin <= CP && W == 32 && H % (PIX / 32) == 0 &&
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
    if (bias) image_fwd_f64_kernel<32, true><<<grid, dim3(NT), 0, c->stream>>>(p);
    else image_fwd_f64_kernel<32, false><<<grid, dim3(NT), 0, c->stream>>>(p);
    FX_LAUNCH_CHECK();
    return FX_OK;
}

}  // namespace cim
