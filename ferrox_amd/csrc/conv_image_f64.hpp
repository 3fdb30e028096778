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

// ---- weight gradient of the same layer (1 to 3 channels: K = Cin * 9 <= 27 <= 32), by row bands ---------------------------------
//   dw[oc][c][ky][kx] = sum over (b, oy, ox) of g[b][oc][oy][ox] * x[b][c][oy + ky - 1][ox + kx - 1]
// (grad_out_2d . im2col(x)^T, convolutions.rs:296-338).  The MFMA's 16 columns are (channel, tap) pairs -- two blocks of 16 hold
// the K <= 27 of them -- and its reduction runs over 4 pixels.  Every WAVE is on its own: it takes a band of rb output rows of one
// image, copies the rb + 2 input rows under it into its private piece of LDS, and feeds g to the MFMA straight from global memory
// -- which pixel goes to which reduction step is free as long as both operands agree: lane (m = l % 16, q = l / 16) takes the 8
// pixels 8 q .. 8 q + 7 of a row as four 16-byte loads per block of 16 output channels, two rows of loads in flight.  No block
// barrier before the closing sum of the four waves (wave order, through LDS); one partial sum per block, laid out like dw, added by
// the ordered split sum.  Bound by the one read of g.  (A block-tile form -- 256 pixels of g staged through LDS behind two barriers
// per tile, blocks in lockstep -- ran [256,3,32,32] -> 32 in 24.7 us, with mask and bias sums 42.3 us; this one 20.7 / 27.0 us.)
// MASK: the gradient arrives unmasked and this layer's ReLU is applied to g as it is loaded (g * (act > 0), the bits of
// fx_relu_bwd); pair index K <= 27 of the 32 is free, and with an operand of 1.0 there the MFMA leaves the sums of the masked g
// over the pixels in it: the bias gradient.
struct RowWParams {
    const double* x;
    const double* g;
    const double* act;
    double* part;
    i64 part_stride;
    int Cin, Cout, H, B;
    int rb, bands, ntasks;
    int PLANE, wave_doubles;  // (rb + 2) * 34 doubles per channel plane; doubles of LDS per wave
    FastDiv div_bands, div_pr;
};
constexpr int NTR = 256, ROW_NPV = 8;  // threads per block; double2 of the patch one lane keeps in flight

template <bool MASK>
__global__ __launch_bounds__(NTR) void image_wgrad_rows_f64_kernel(const RowWParams p) {
    constexpr int W = 32, PW = W + 2, W2 = W / 2;
    FX_DYNAMIC_SMEM(double, smem_r);
    const int tid = threadIdx.x, lane = tid & 63, kq = lane >> 4, l16 = lane & 15;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int task = blockIdx.x * 4 + wave;
    double* patch = smem_r + wave * p.wave_doubles;
    const int oc0 = blockIdx.y * 32, L = p.H * W, K = p.Cin * KK;
    int xoff[2];
    bool pair_ok[2], pair_one[2];
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
        const int kp = 16 * nb + l16;
        pair_ok[nb] = kp < K;
        pair_one[nb] = MASK && kp == K;
        const int c = pair_ok[nb] ? kp / KK : 0, t = pair_ok[nb] ? kp % KK : 0;
        xoff[nb] = c * p.PLANE + (t / 3) * PW + t % 3 + 8 * kq;  // pixel (row 0, column 8 q): + PW per row, + j per step
    }
    f64x4 acc[2][2];  // [oc block][pair block]
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[m][nb][e] = 0.;
    if (task < p.ntasks) {  // wave-uniform
        const int b = (int)p.div_bands.div((uint32_t)task), oy0 = (task - b * p.bands) * p.rb;
        const int nr = min(p.rb, p.H - oy0);
        // lane's 8 pixels of output channel oc0 + 16 m + l16, row oy0 + r: four double2 per m
        const i64 grow = ((i64)b * p.Cout + oc0 + l16) * L + (i64)oy0 * W + 8 * kq;
        double2 gv[2][8], av[2][8];
        auto load = [&](int set, int r) __attribute__((always_inline)) {
#pragma unroll
            for (int m = 0; m < 2; ++m)
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const i64 off = grow + (i64)m * 16 * L + (i64)r * W + 2 * u;
                    gv[set][4 * m + u] = *reinterpret_cast<const double2*>(p.g + off);
                    if constexpr (MASK) av[set][4 * m + u] = *reinterpret_cast<const double2*>(p.act + off);
                }
        };
        auto mul = [&](int set, int r) __attribute__((always_inline)) {
            const double* src = patch + r * PW;
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                double2 g0 = gv[set][u], g1 = gv[set][4 + u];
                if constexpr (MASK) {
                    const double2 a0 = av[set][u], a1 = av[set][4 + u];
                    g0.x = g0.x * (a0.x > 0. ? 1. : 0.); g0.y = g0.y * (a0.y > 0. ? 1. : 0.);
                    g1.x = g1.x * (a1.x > 0. ? 1. : 0.); g1.y = g1.y * (a1.y > 0. ? 1. : 0.);
                }
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const double a0 = j ? g0.y : g0.x, a1 = j ? g1.y : g1.x;
                    double b0 = src[xoff[0] + 2 * u + j], b1 = src[xoff[1] + 2 * u + j];
                    if (!pair_ok[0]) b0 = pair_one[0] ? 1. : 0.;
                    if (!pair_ok[1]) b1 = pair_one[1] ? 1. : 0.;
                    acc[0][0] = __builtin_amdgcn_mfma_f64_16x16x4f64(a0, b0, acc[0][0], 0, 0, 0);
                    acc[0][1] = __builtin_amdgcn_mfma_f64_16x16x4f64(a0, b1, acc[0][1], 0, 0, 0);
                    acc[1][0] = __builtin_amdgcn_mfma_f64_16x16x4f64(a1, b0, acc[1][0], 0, 0, 0);
                    acc[1][1] = __builtin_amdgcn_mfma_f64_16x16x4f64(a1, b1, acc[1][1], 0, 0, 0);
                }
            }
        };
        load(0, 0);
        // the rows [oy0 - 1, oy0 + rb] of the Cin planes into the wave's patch, zero above and below the image and in columns 0 and 33
        {
            const int PR = p.rb + 2, items = p.Cin * PR * W2;
            const double* xsrc = p.x + (i64)b * p.Cin * L;
            double2 v[ROW_NPV];
            int dst[ROW_NPV];
#pragma unroll
            for (int u = 0; u < ROW_NPV; ++u) {
                const int i = min(lane + 64 * u, items - 1);
                const int rc = i / W2, q2 = i - rc * W2;
                const int c = (int)p.div_pr.div((uint32_t)rc), r = rc - c * PR;
                const int iy = oy0 - 1 + r;
                const bool ok = iy >= 0 && iy < p.H;
                v[u] = *reinterpret_cast<const double2*>(xsrc + ((i64)c * p.H + (ok ? iy : 0)) * W + 2 * q2);
                if (!ok) v[u] = make_double2(0., 0.);
                dst[u] = c * p.PLANE + r * PW + 1 + 2 * q2;
            }
            for (int i = lane; i < p.Cin * PR; i += 64) {
                const int c = (int)p.div_pr.div((uint32_t)i), r = i - c * PR;
                patch[c * p.PLANE + r * PW] = 0.;
                patch[c * p.PLANE + r * PW + W + 1] = 0.;
            }
#pragma unroll
            for (int u = 0; u < ROW_NPV; ++u)
                if (lane + 64 * u < items) {
                    double* d = patch + dst[u];
                    d[0] = v[u].x;
                    d[1] = v[u].y;
                }
            __builtin_amdgcn_wave_barrier();  // one wave: its LDS accesses complete in program order, so this is a scheduling fence only
        }
        for (int r = 0; r < nr; r += 2) {
            if (r + 1 < nr) load(1, r + 1);
            mul(0, r);
            if (r + 2 < nr) load(0, r + 2);
            if (r + 1 < nr) mul(1, r + 1);
        }
    }
    // the four waves hold sums over different bands: added in wave order (the patches are dead after the barrier)
    __syncthreads();
    double* red = smem_r;  // [4 waves][16 elements][64 lanes]
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
    for (int u = 0; u < 4; ++u) {
        const int el = 4 * wave + u, blk = el >> 2, e = el & 3;  // wave w finishes elements 4 w .. 4 w + 3
        const double v = ((red[el * 64 + lane] + red[(16 + el) * 64 + lane]) + red[(32 + el) * 64 + lane]) + red[(48 + el) * 64 + lane];
        const int oc = 16 * (blk >> 1) + 4 * e + kq, kp = 16 * (blk & 1) + l16;
        if (kp < K) out[(i64)oc * K + kp] = v;
        if (MASK && kp == K) bout[oc] = v;
    }
}

struct WPlan {
    bool ok = false;
    int rb = 0, tasks = 0, splits = 1;  // rows per band, bands in all, blocks (= partial sums)
    i64 B = 0;
};

inline WPlan wgrad_plan(int num_cus, i64 B, i64 Cin, i64 H, i64 W, i64 Cout, i64 kh, i64 kw, i64 sh, i64 sw, i64 ph, i64 pw) {
    WPlan pl;
    if (kh != 3 || kw != 3 || sh != 1 || sw != 1 || ph != 1 || pw != 1 || Cin < 1 || Cin > 3 || W != 32 || Cout % 32 != 0)
        return pl;
    const i64 rows = Cout / 32;
    if (rows > 65535 || B * H > 0x3fffffff) return pl;
    pl.B = B;
    // about one wave per SIMD (measured for the f32 twin of this kernel, conv_smallc.hpp), within what a lane stages
    i64 rb = std::max<i64>(2, std::min<i64>(8, B * H / (4 * (i64)std::max(1, num_cus))));
    rb = std::min<i64>(rb, H);
    while (rb > 1 && Cin * (rb + 2) * 16 > ROW_NPV * 64) --rb;
    if (Cin * (rb + 2) * 16 > ROW_NPV * 64) return pl;
    pl.rb = (int)rb;
    pl.tasks = (int)(B * fx::ceil_div(H, rb));
    pl.splits = (int)fx::ceil_div((i64)pl.tasks, (i64)4);
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
    RowWParams q;
    q.x = x; q.g = g; q.act = act; q.part = part;
    q.part_stride = Cout * Cin * KK + (act ? Cout : 0);
    q.Cin = (int)Cin; q.Cout = (int)Cout; q.H = (int)H; q.B = (int)pl.B;
    q.rb = pl.rb; q.bands = (int)fx::ceil_div(H, (i64)pl.rb); q.ntasks = pl.tasks;
    q.PLANE = (pl.rb + 2) * 34;
    q.wave_doubles = (int)Cin * q.PLANE;
    q.div_bands = FastDiv((uint32_t)q.bands); q.div_pr = FastDiv((uint32_t)(pl.rb + 2));
    const size_t lds = std::max((size_t)4 * q.wave_doubles, (size_t)4 * 16 * 64) * sizeof(double);
    const dim3 grid((unsigned)pl.splits, (unsigned)(Cout / 32));
    if (act) FX_LAUNCH(grid, dim3(NTR), lds, c->stream, (q), image_wgrad_rows_f64_kernel<true>);
    else FX_LAUNCH(grid, dim3(NTR), lds, c->stream, (q), image_wgrad_rows_f64_kernel<false>);
    FX_LAUNCH_CHECK();
    if (act) return igemm::launch_splitk_reduce_pair<double>(c, part, q.part_stride, pl.splits, dw, Cout * Cin * KK, db, Cout);
    return igemm::launch_splitk_reduce<double>(c, part, dw, Cout * Cin * KK, pl.splits);
}

}  // namespace cim
