// Weight gradient of a 3x3 convolution of stride 2 and padding 1 over an even-sized map (f64): the twin of
// wg2::wgrad_s2_kernel (wgrad_patch_s2.hpp) on v_mfma_f64_16x16x4_f64, same product
//   dw[oc][c][ky][kx] = sum over (b, oy, ox) of g[b][oc][oy][ox] * x[b][c][2 oy + ky - 1][2 ox + kx - 1]
// (grad_out_2d . im2col(x)^T in the reference, src/backend/storage/extensions/convolutions.rs:296-338).
//
// The f64 MFMA adds a 16(oc) x 4(pixel) by 4(pixel) x 16(c) product to a 16 x 16 block: lane l holds g[oc = l % 16][pixel + l / 16]
// and x[c = l % 16][that pixel's tap], one double each, and 4 of the 256 sums (oc = 4 e + l / 16, c = l % 16).
// One block per CU (4 waves, all 512 registers of a lane, accumulators in the accumulation registers) takes 64 output
// channels x 32 input channels; its waves are laid out 2 x 2 -- 32 output channels x 16 input channels each, 2 x 9
// accumulator blocks (one per tap: 144 registers) -- and every wave runs all pixels of a stage, so no sums are exchanged
// between waves.  A stage is R output rows of one image (32 pixels, 2 R + 1 patch rows), in two LDS buffers: the next stage
// is loaded into registers before the MFMA loop of the current one and parked after it, one barrier per stage.
//   Gs[oc][pixel]      64 output-channel rows of g, the stage's pixels contiguous as in memory  (odd pitch GP)
//   Xs[c][row][col]    32 input-channel planes of the zero-padded patch rows                    (odd pitch PLANE)
// Per group of 4 pixels a wave reads 2 values of g and 9 of the patch for 18 MFMAs, every LDS address a per-lane base plus an
// immediate.  Blocks over disjoint stage ranges leave partial sums ([oc][tap][c]) that wgd's reduce kernel adds in order.
#pragma once
#include <cstdlib>

#include "wgrad_patch_f64.hpp"

namespace wgd2 {
using igemm::FastDiv;
using igemm::f64x4;
using wgd::ldg2;

constexpr int KK = 9, NT = 256, BM = 64, CT = 32;
constexpr size_t LDS_LIMIT = 160 * 1024;

struct Params {
    const double* x;
    const double* g;
    const double* act;  // MASK: the layer's ReLU output; g is staged as g * (act > 0)
    double* part;
    double* bpart;      // MASK: per-split sums of the masked g per output channel ([Cout], part_stride apart): the bias gradient
    int Cin, H, Cout, oh, ph;
    int stages, sps, spi;  // all stages, stages per split, stages per image
    int xcd_chunk;         // blocks / 8 when that divides, else 0
    FastDiv div_spi;
    i64 part_stride;
};

template <int OW, int R>
struct Shape {
    static constexpr int W = 2 * OW, PW = W + 2, XR = 2 * R + 1;
    static constexpr int KST = R * OW;                                    // pixels per stage
    static constexpr int GP = KST | 1, PLANE = (XR * PW) | 1;
    static constexpr int XL = W / 2, RX = NT / XL;                        // lanes per patch row, (row, channel) pairs per pass
    static constexpr int NXP = XR * CT / RX;                              // passes over the pairs, row-major
    static constexpr int GL = KST / 2, GR = NT / GL;                      // lanes per row of g, rows per pass
    static constexpr int NG = BM / GR;
    static constexpr int GROUPS = KST / 4, GPR = OW / 4;                  // groups of 4 pixels per stage, per output row
    static constexpr int BUF = BM * GP + CT * PLANE;                      // doubles per stage buffer
    static constexpr size_t LDS = 2 * (size_t)BUF * sizeof(double);
    static_assert(OW % 4 == 0 && NT % XL == 0 && CT % RX == 0 && XR * CT % RX == 0 && NT % GL == 0 && BM % GR == 0 && LDS <= LDS_LIMIT, "shape");
    static_assert(GL == 16, "the bias sums of the masked variant are added over the 16 lanes of a row");
};

// MASK: the gradient arrives unmasked from the layer above; the ReLU of this layer is applied to the staged rows of g
// (g * (act > 0), the bits of fx_relu_bwd) and the blocks of the first channel tile also leave the sums of the masked rows
// over their stages: the bias gradient.
template <int OW, int R, bool MASK>
__global__ __launch_bounds__(NT, 1) void wgrad_s2_f64_kernel(const Params p) {
    using S = Shape<OW, R>;
    constexpr int W = S::W, PW = S::PW, GP = S::GP, PLANE = S::PLANE, BUF = S::BUF;
    FX_DYNAMIC_SMEM(double, smem_wgd2);
    double* smem = smem_wgd2;
    const int tid = threadIdx.x, lane = tid & 63, kq = lane >> 4, l16 = lane & 15;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wmo = wave & 1, wc = wave >> 1;
    // Workgroup ids go to the 8 XCDs round-robin; remapped so that each XCD takes a contiguous range of (split, oc tile,
    // channel tile) triples: the tiles of one split read the same rows of g and x through one L2.
    int bxi = blockIdx.x, byi = blockIdx.y, bzi = blockIdx.z;
    if (p.xcd_chunk) {
        const int lin = bxi + gridDim.x * (byi + gridDim.y * bzi);
        const int id = (lin & 7) * p.xcd_chunk + (lin >> 3);
        bxi = id % gridDim.x;
        const int rest = id / gridDim.x;
        byi = rest % gridDim.y;
        bzi = rest / gridDim.y;
    }
    const int c0 = bxi * CT, oc0 = byi * BM;
    const int L = p.oh * OW;
    {
        // one wave per SIMD owns all 512 registers of a lane: once a function touches the accumulation registers the compiler
        // splits them 256 + 256 and keeps the MFMA accumulators there
        int z = 0;
        FX_TOUCH_AGPR(z);
    }
    f64x4 acc[2][KK];
#pragma unroll
    for (int o = 0; o < 2; ++o)
#pragma unroll
        for (int t = 0; t < KK; ++t)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[o][t][e] = 0.;

    // Staging.  g: thread t owns double2 column t % GL of rows t / GL + GR u.  x: the (patch row, channel) pairs are numbered
    // row-major, q = 32 r + c; thread t owns double2 column t % XL of pairs t / XL + RX u, so the patch row of a pass is a
    // compile-time constant and its validity a scalar.
    const double2 zero2 = make_double2(0., 0.);
    double2 gv[S::NG], xv[S::NXP], av[MASK ? S::NG : 1];
    double bsum[S::NG];
#pragma unroll
    for (int u = 0; u < S::NG; ++u) bsum[u] = 0.;
    const int gq = tid % S::GL, grow = tid / S::GL;
    const int xq = tid % S::XL, xrow = tid / S::XL;
    const uint32_t g_off = (uint32_t)(grow * L + 2 * gq) * 8u;
    const uint32_t x_off = (uint32_t)(xrow * p.H * W + 2 * xq) * 8u;
    const int g_dst0 = grow * GP + 2 * gq;
    const int x_dst0 = BM * GP + xrow * PLANE + 1 + 2 * xq;
    auto prefetch = [&](int s) __attribute__((always_inline)) {
        const int b = (int)p.div_spi.div((uint32_t)s);
        const int oy0 = (s - b * p.spi) * R;
        const int iy0 = 2 * oy0 - p.ph;
        const double* gsrc = p.g + ((i64)b * p.Cout + oc0) * L + (i64)oy0 * OW;
        const double* xsrc = p.x + ((i64)b * p.Cin + c0) * p.H * W;
#pragma unroll
        for (int u = 0; u < S::NG; ++u) gv[u] = ldg2(gsrc + (i64)u * S::GR * L, g_off);
        if constexpr (MASK) {
            const double* asrc = p.act + ((i64)b * p.Cout + oc0) * L + (i64)oy0 * OW;
#pragma unroll
            for (int u = 0; u < S::NG; ++u) av[u] = ldg2(asrc + (i64)u * S::GR * L, g_off);
        }
#pragma unroll
        for (int u = 0; u < S::NXP; ++u) {
            const int r = u * S::RX / CT, cb = u * S::RX % CT;  // patch row and first channel of this pass
            const int iy = iy0 + r;
            if (iy >= 0 && iy < p.H) xv[u] = ldg2(xsrc + ((i64)cb * p.H + iy) * W, x_off);  // scalar condition
            else xv[u] = zero2;
        }
    };
    auto park = [&](int buf) __attribute__((always_inline)) {
        int gd = g_dst0 + buf * BUF, xd = x_dst0 + buf * BUF;
        FX_PIN_VGPR2(gd, xd);
#pragma unroll
        for (int u = 0; u < S::NG; ++u) {
            double* d = smem + gd + u * S::GR * GP;
            if constexpr (MASK) {
                gv[u].x = gv[u].x * (av[u].x > 0. ? 1. : 0.);
                gv[u].y = gv[u].y * (av[u].y > 0. ? 1. : 0.);
                bsum[u] = bsum[u] + (gv[u].x + gv[u].y);
            }
            d[0] = gv[u].x; d[1] = gv[u].y;
        }
#pragma unroll
        for (int u = 0; u < S::NXP; ++u) {
            const int r = u * S::RX / CT, cb = u * S::RX % CT;
            double* d = smem + xd + cb * PLANE + r * PW;
            d[0] = xv[u].x; d[1] = xv[u].y;
        }
    };

    // One stage: GROUPS groups of 4 pixels.  Lane l holds g[oc = l % 16 (+ 16)][pixel + l / 16] and, for tap (ky, kx),
    // x[c = l % 16][2 (pixel + l / 16) + (ky, kx)]; the operands of a group are read while the 18 MFMAs of the group before run.
    const int ga0 = (wmo * 32 + l16) * GP + kq;
    const int xb0 = BM * GP + (wc * 16 + l16) * PLANE + 2 * kq;
    auto compute = [&](int buf) __attribute__((always_inline)) {
        const double* ga = smem + ga0 + buf * BUF;
        const double* xb = smem + xb0 + buf * BUF;
        constexpr int U = S::GROUPS;
        double a[U][2], b[U][KK];
        auto rd = [&](int u) __attribute__((always_inline)) {
            const int r = u / S::GPR, j = u % S::GPR;
            a[u][0] = ga[r * OW + 4 * j];
            a[u][1] = ga[16 * GP + r * OW + 4 * j];
#pragma unroll
            for (int ky = 0; ky < 3; ++ky)
#pragma unroll
                for (int kx = 0; kx < 3; ++kx) b[u][ky * 3 + kx] = xb[(2 * r + ky) * PW + 8 * j + kx];
            __builtin_amdgcn_sched_barrier(0);
        };
        rd(0);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (u + 1 < U) rd(u + 1);
#pragma unroll
            for (int t = 0; t < KK; ++t)
#pragma unroll
                for (int o = 0; o < 2; ++o) acc[o][t] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[u][o], b[u][t], acc[o][t], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    const int s_beg = bzi * p.sps, s_end = min(p.stages, s_beg + p.sps);
    if (s_beg < s_end) prefetch(s_beg);
    // Column 0 of every patch row is the zero padding left of the image: written once in both buffers.  The staged columns
    // 1 .. W are rewritten by every stage (rows above and below the image as zeros); column W + 1 is never read.
    for (int i = tid; i < 2 * CT * S::XR; i += NT) {
        const int buf = i / (CT * S::XR), rem = i - buf * (CT * S::XR), c = rem / S::XR, r = rem - c * S::XR;
        smem[buf * BUF + BM * GP + c * PLANE + r * PW] = 0.;
    }
    if (s_beg < s_end) park(0);
    __syncthreads();
    int cur = 0;
    for (int s = s_beg; s < s_end; ++s) {
        const bool more = s + 1 < s_end;
        if (more) prefetch(s + 1);
        compute(cur);
        // the other buffer was last read in the stage before this one, which every wave has left through the barrier below
        if (more) park(cur ^ 1);
        __syncthreads();
        cur ^= 1;
    }

    if constexpr (MASK) {
        // bias gradient of this block's stages: the 16 lanes that share a row of g add their sums in a fixed butterfly order
        if (bxi == 0) {
#pragma unroll
            for (int u = 0; u < S::NG; ++u) {
                double v = bsum[u];
                v = v + __shfl_xor(v, 8, 64);
                v = v + __shfl_xor(v, 4, 64);
                v = v + __shfl_xor(v, 2, 64);
                v = v + __shfl_xor(v, 1, 64);
                if (gq == 0) p.bpart[(i64)bzi * p.part_stride + oc0 + grow + S::GR * u] = v;
            }
        }
    }
    double* out = p.part + (i64)bzi * p.part_stride;
    const int ldo = KK * p.Cin;
#pragma unroll
    for (int o = 0; o < 2; ++o)
#pragma unroll
        for (int t = 0; t < KK; ++t)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int oc = oc0 + wmo * 32 + o * 16 + igemm::Mfma<double>::row(e, lane);
                out[(i64)oc * ldo + t * p.Cin + c0 + wc * 16 + l16] = acc[o][t][e];
            }
}

struct Plan {
    bool ok = false;
    int OW = 0, R = 0, splits = 1, sps = 1, stages = 0;
    size_t smem = 0;
};

// Instantiated (OW, R): rows of 16 and 32 pixels (maps 32 and 64 wide), 32 pixels per stage.
#define FX_WGD2_SHAPES(X) X(16, 2) X(32, 1) X(8, 4)

inline Plan make_plan(int num_cus, i64 B, i64 Cin, i64 H, i64 W, i64 Cout, i64 kh, i64 kw, i64 sh, i64 sw, i64 ph, i64 pw, i64 oh, i64 ow) {
    Plan pl;
    if (kh != 3 || kw != 3 || sh != 2 || sw != 2 || pw != 1 || ph > 1 || W != 2 * ow || Cin % CT != 0 || Cout % BM != 0) return pl;
    if (Cout * Cin * KK > 0x7fffffff || 32 * H * W * 8 > 0x7fffffff || Cout * oh * ow * 8 > 0x7fffffff) return pl;
#define FX_WGD2_PICK(O, RR)                                              \
    if (!pl.ok && ow == O && oh % RR == 0) {                             \
        pl.ok = true; pl.OW = O; pl.R = RR;                              \
        pl.smem = Shape<O, RR>::LDS;                                     \
    }
    FX_WGD2_SHAPES(FX_WGD2_PICK)
#undef FX_WGD2_PICK
    if (!pl.ok) return pl;
    pl.ok = false;
    pl.stages = (int)(B * (oh / pl.R));
    const i64 tiles = (Cin / CT) * (Cout / BM);
    // one block per CU; at least two stages per block where there are that many (a block's partial sum is paid once)
    const i64 splits = std::max<i64>(1, std::min<i64>((i64)num_cus / tiles, std::max<i64>(1, pl.stages / 2)));
    pl.sps = (int)fx::ceil_div((i64)pl.stages, splits);
    pl.splits = (int)fx::ceil_div((i64)pl.stages, (i64)pl.sps);
    if (pl.splits > 65535 || tiles > 65535 || B * oh > 0x7fffffff) return pl;
    pl.ok = true;
    return pl;
}

// the masked variant keeps [Cout] bias sums behind every split's partial
inline i64 workspace_bytes(const Plan& pl, i64 Cout, i64 Cin, bool with_bias = false) {
    return (i64)pl.splits * (Cout * Cin * KK + (with_bias ? Cout : 0)) * (i64)sizeof(double);
}

// x, g and part must be 16-byte aligned.
// act / db non-null: the masked variant (act 16-byte aligned as well).
inline int run(fx_ctx* c, const Plan& pl, const double* x, const double* g, double* dw, double* part, i64 Cin, i64 H, i64 Cout, i64 ph, i64 oh,
               const double* act = nullptr, double* db = nullptr) {
    Params p;
    p.x = x; p.g = g; p.part = part; p.act = act; p.bpart = part + Cout * Cin * KK;
    p.Cin = (int)Cin; p.H = (int)H; p.Cout = (int)Cout; p.oh = (int)oh; p.ph = (int)ph;
    p.stages = pl.stages; p.sps = pl.sps; p.spi = (int)(oh / pl.R);
    p.div_spi = FastDiv((uint32_t)p.spi);
    p.part_stride = Cout * Cin * KK + (act ? Cout : 0);
    const dim3 grid((unsigned)(Cin / CT), (unsigned)(Cout / BM), (unsigned)pl.splits);
    const i64 blocks = (i64)grid.x * grid.y * grid.z;
    p.xcd_chunk = blocks % 8 == 0 && blocks <= 0x7fffffff ? (int)(blocks / 8) : 0;
    bool launched = false;
#define FX_WGD2_LAUNCH(O, RR)                                                                                          \
    if (!launched && pl.OW == O && pl.R == RR) {                                                                       \
        static const hipError_t attr = hipFuncSetAttribute((const void*)wgrad_s2_f64_kernel<O, RR, false>,             \
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_LIMIT); \
        static const hipError_t attr_m = hipFuncSetAttribute((const void*)wgrad_s2_f64_kernel<O, RR, true>,            \
                                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_LIMIT); \
        FX_HIP_CHECK(attr);                                                                                            \
        FX_HIP_CHECK(attr_m);                                                                                          \
        if (act) FX_LAUNCH(grid, dim3(NT), pl.smem, c->stream, (p), wgrad_s2_f64_kernel<O, RR, true>);                          \
        else FX_LAUNCH(grid, dim3(NT), pl.smem, c->stream, (p), wgrad_s2_f64_kernel<O, RR, false>);                             \
        launched = true;                                                                                               \
    }
    FX_WGD2_SHAPES(FX_WGD2_LAUNCH)
#undef FX_WGD2_LAUNCH
    FX_REQUIRE(launched, "wgrad stride-2 patch kernel (f64): unexpected shape (%d, %d)", pl.OW, pl.R);
    FX_LAUNCH_CHECK();
    const int n = (int)(Cout * Cin * KK);
    const wgd::ReduceTail tail{p.part_stride, act ? db : nullptr, act ? (int)Cout : 0};
    const FastDiv div_row((uint32_t)(KK * Cin)), div_cin((uint32_t)Cin);
    // many partials of a small output: the grouped 16-byte sum (n, Cin and the stride are even here, part is 16-byte aligned)
    if (pl.splits >= 64 && n <= (1 << 18))
        FX_LAUNCH(dim3((unsigned)(fx::ceil_div((i64)n, 32) + wgd::tail_blocks(tail, 16))), dim3(256), 0, c->stream, (part, dw, n, pl.splits, (int)Cin, div_row, div_cin, tail), wgd::wgrad_f64_reduce_vec_kernel<16>);
    else
        FX_LAUNCH(dim3((unsigned)(fx::ceil_div((i64)n, 256) + wgd::tail_blocks(tail, 256))), dim3(256), 0, c->stream, (part, dw, n, pl.splits, (int)Cin, div_row, div_cin, tail), wgd::wgrad_f64_reduce_kernel);
    FX_LAUNCH_CHECK();
    return FX_OK;
}

}  // namespace wgd2
