// Weight gradient of a 3x3 convolution of stride 2 and padding 1 over an even-sized map (f32): the stride-2 member of the
// family of wgp::wgrad_patch_kernel (wgrad_patch.hpp), same product
//   dw[oc][c][ky][kx] = sum over (b, oy, ox) of g[b][oc][oy][ox] * x[b][c][2 oy + ky - 1][2 ox + kx - 1]
// (grad_out_2d . im2col(x)^T in the reference, src/backend/storage/extensions/convolutions.rs:296-338).
//
// A strided layer has four input values per output pixel, so a stage of the same pixel count stages four times the patch
// of a unit-stride layer and the reduction per CU is short (the layers are small).  This kernel therefore takes one block
// per CU with all 512 registers of a lane (accumulators in the accumulation registers), R output rows of one image per
// stage (2 R + 1 patch rows), and two stage buffers in LDS: the next stage's operands are parked while other waves still
// compute, and a stage costs one barrier.  The row length is a compile-time constant, so every LDS read of the unrolled
// pixel loop is a per-lane base plus an immediate:
//   Gs[oc][pixel]      BM = 32 WMO output-channel rows of g, the stage's R OW pixels contiguous as in memory (pitch GP)
//   Xs[c][row][col]    32 input-channel planes of the zero-padded patch rows                               (pitch PLANE)
// both pitches = 1 mod 32, so the 32 lanes of a half-wave read 32 different banks.  The four waves are WMO blocks of 32
// output channels x WK = 4 / WMO segments of every pixel row; a wave runs 9 accumulator blocks of 32(oc) x 32(c), one per
// tap, and per pixel pair reads 1 value of g and 9 of the patch for its 9 MFMAs.  The segments' sums are added in order when
// the block ends; blocks over disjoint stage ranges leave partial sums ([oc][tap][c]) that wgp's reduce kernels add in order.
#pragma once
#include <cstdlib>

#include "wgrad_patch.hpp"

namespace wg2 {
using igemm::FastDiv;
using igemm::f32x16;
using igemm::ldg4;

constexpr int KK = 9, NT = 256, CT = 32;
constexpr size_t LDS_LIMIT = 160 * 1024;

constexpr int odd_pitch(int n) { return (n + 30) / 32 * 32 + 1; }
// position of tap t among the taps that the wave of segment q hands over (those with t' % WK != q)
constexpr int slot(int t, int q, int wk) {
    int n = 0;
    for (int u = 0; u < t; ++u) n += u % wk != q;
    return n;
}

struct Params {
    const float* x;
    const float* g;
    const float* act;  // MASK: the layer's ReLU output; g is staged as g * (act > 0)
    float* part;
    float* bpart;      // MASK: per-split sums of the masked g per output channel ([Cout], part_stride apart): the bias gradient
    int Cin, H, Cout, oh, ph;
    int stages, sps, spi;  // all stages, stages per split, stages per image
    int xcd_chunk;         // blocks / 8 when that divides, else 0
    FastDiv div_spi;
    i64 part_stride;
};

template <int WMO, int OW, int R>
struct Shape {
    static constexpr int WK = 4 / WMO, BM = 32 * WMO;
    static constexpr int W = 2 * OW, PW = W + 2, XR = 2 * R + 1;
    static constexpr int KST = R * OW;                                    // pixels per stage
    static constexpr int GP = odd_pitch(KST), PLANE = odd_pitch(XR * PW);
    static constexpr int XL = W <= 32 ? 8 : 16, RX = NT / XL;             // lanes per patch row, patch rows per pass of the block
    static constexpr int NXP = XR * CT / RX;                              // passes over the (row, channel) pairs, row-major
    static constexpr int NG = BM / 16;                                    // passes over the rows of g, 16 lanes per row
    static constexpr int SEG = OW / WK, PAIRS = SEG / 2;
    static constexpr int BUF = BM * GP + CT * PLANE;                      // floats per stage buffer
    static constexpr int NS = KK - KK / WK;                               // most taps a wave hands over in the closing sum
    static constexpr size_t RED = WK == 2 ? (size_t)4 * NS * 16 * 64 * sizeof(float) : (size_t)4 * 16 * 64 * sizeof(float);
    static constexpr size_t LDS = 2 * (size_t)BUF * sizeof(float) > RED ? 2 * (size_t)BUF * sizeof(float) : RED;
    static_assert(WMO * WK == 4 && SEG % 2 == 0 && KST % 4 == 0 && KST <= 64 && W % 4 == 0 && W / 4 <= XL, "shape");
    static_assert(XR * CT % RX == 0 && LDS <= LDS_LIMIT, "staging");
};

// MASK: the gradient arrives unmasked from the layer above; the ReLU of this layer is applied to the staged rows of g
// (g * (act > 0), the bits of fx_relu_bwd) and the blocks of the first channel tile also leave the sums of the masked rows
// over their stages -- the bias gradient -- so no masked copy of g and no separate bias pass exist.
template <int WMO, int OW, int R, bool MASK>
__global__ __launch_bounds__(NT, 1) void wgrad_s2_kernel(const Params p) {
    using S = Shape<WMO, OW, R>;
    constexpr int WK = S::WK, BM = S::BM, W = S::W, PW = S::PW, GP = S::GP, PLANE = S::PLANE, BUF = S::BUF;
    FX_DYNAMIC_SMEM(float, smem);
    const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5, l32 = lane & 31;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wmo = wave % WMO, wk = wave / WMO;
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
    f32x16 acc[KK];
#pragma unroll
    for (int t = 0; t < KK; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[t][e] = 0.f;

    // Staging.  g: thread t owns float4 column t % 16 of rows t / 16 + 16 u.  x: the (patch row, channel) pairs are numbered
    // row-major, q = 32 r + c; thread t owns float4 column t % XL of pairs t / XL + RX u, so the patch row of a pass is a
    // compile-time constant and its validity a scalar.
    const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
    float4 gv[S::NG], xv[S::NXP], av[MASK ? S::NG : 1];
    float bsum[S::NG];
#pragma unroll
    for (int u = 0; u < S::NG; ++u) bsum[u] = 0.f;
    const int gq = tid & 15, grow = tid >> 4;
    const int xq = tid & (S::XL - 1), xrow = tid / S::XL;
    const bool g_lane = gq < S::KST / 4, x_lane = xq < W / 4;
    const uint32_t g_off = (uint32_t)(grow * L + (g_lane ? 4 * gq : 0)) * 4u;
    const uint32_t x_off = (uint32_t)(xrow * p.H * W + (x_lane ? 4 * xq : 0)) * 4u;
    const int g_dst0 = grow * GP + 4 * gq;
    const int x_dst0 = BM * GP + xrow * PLANE + 1 + 4 * xq;
    auto prefetch = [&](int s) __attribute__((always_inline)) {
        const int b = (int)p.div_spi.div((uint32_t)s);
        const int oy0 = (s - b * p.spi) * R;
        const int iy0 = 2 * oy0 - p.ph;
        const float* gsrc = p.g + ((i64)b * p.Cout + oc0) * L + (i64)oy0 * OW;
        const float* xsrc = p.x + ((i64)b * p.Cin + c0) * p.H * W;
#pragma unroll
        for (int u = 0; u < S::NG; ++u) gv[u] = ldg4(gsrc + (i64)u * 16 * L, g_off);
        if constexpr (MASK) {
            const float* asrc = p.act + ((i64)b * p.Cout + oc0) * L + (i64)oy0 * OW;
#pragma unroll
            for (int u = 0; u < S::NG; ++u) av[u] = ldg4(asrc + (i64)u * 16 * L, g_off);
        }
#pragma unroll
        for (int u = 0; u < S::NXP; ++u) {
            const int r = u * S::RX / CT, cb = u * S::RX % CT;  // patch row and first channel of this pass
            const int iy = iy0 + r;
            if (iy >= 0 && iy < p.H) xv[u] = ldg4(xsrc + ((i64)cb * p.H + iy) * W, x_off);  // scalar condition
            else xv[u] = zero4;
        }
    };
    auto park = [&](int buf) __attribute__((always_inline)) {
        int gd = g_dst0 + buf * BUF, xd = x_dst0 + buf * BUF;
        FX_PIN_VGPR2(gd, xd);
        if (g_lane) {
#pragma unroll
            for (int u = 0; u < S::NG; ++u) {
                float* d = smem + gd + u * 16 * GP;
                if constexpr (MASK) {
                    gv[u].x = gv[u].x * (av[u].x > 0.f ? 1.f : 0.f); gv[u].y = gv[u].y * (av[u].y > 0.f ? 1.f : 0.f);
                    gv[u].z = gv[u].z * (av[u].z > 0.f ? 1.f : 0.f); gv[u].w = gv[u].w * (av[u].w > 0.f ? 1.f : 0.f);
                    bsum[u] = bsum[u] + ((gv[u].x + gv[u].y) + (gv[u].z + gv[u].w));
                }
                d[0] = gv[u].x; d[1] = gv[u].y; d[2] = gv[u].z; d[3] = gv[u].w;
            }
        }
        if (x_lane) {
#pragma unroll
            for (int u = 0; u < S::NXP; ++u) {
                const int r = u * S::RX / CT, cb = u * S::RX % CT;
                float* d = smem + xd + cb * PLANE + r * PW;
                d[0] = xv[u].x; d[1] = xv[u].y; d[2] = xv[u].z; d[3] = xv[u].w;
            }
        }
    };

    // One stage: R rows x PAIRS pixel pairs per wave.  Lane l holds g[oc = l % 32][pixel + l / 32] and, for tap (ky, kx),
    // x[c = l % 32][2 (pixel + l / 32) + (ky, kx)]; the operands of a pair are read while the 9 MFMAs of the pair before run.
    const int ga0 = (wmo * 32 + l32) * GP + wk * S::SEG + half;
    const int xb0 = BM * GP + l32 * PLANE + 2 * (wk * S::SEG + half);
    auto compute = [&](int buf) __attribute__((always_inline)) {
        const float* ga = smem + ga0 + buf * BUF;
        const float* xb = smem + xb0 + buf * BUF;
        constexpr int U = R * S::PAIRS;
        float a[U], b[U][KK];
        auto rd = [&](int u) __attribute__((always_inline)) {
            const int r = u / S::PAIRS, j = u % S::PAIRS;
            a[u] = ga[r * OW + 2 * j];
#pragma unroll
            for (int ky = 0; ky < 3; ++ky)
#pragma unroll
                for (int kx = 0; kx < 3; ++kx) b[u][ky * 3 + kx] = xb[(2 * r + ky) * PW + 4 * j + kx];
            __builtin_amdgcn_sched_barrier(0);
        };
        rd(0);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (u + 1 < U) rd(u + 1);
#pragma unroll
            for (int t = 0; t < KK; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u], b[u][t], acc[t], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    const int s_beg = bzi * p.sps, s_end = min(p.stages, s_beg + p.sps);
    if (s_beg < s_end) prefetch(s_beg);
    // Column 0 of every patch row is the zero padding left of the image: written once in both buffers.  The staged columns
    // 1 .. W are rewritten by every stage (rows above and below the image as zeros); column W + 1 is never read.
    for (int i = tid; i < 2 * CT * S::XR; i += NT) {
        const int buf = i / (CT * S::XR), rem = i - buf * (CT * S::XR), c = rem / S::XR, r = rem - c * S::XR;
        smem[buf * BUF + BM * GP + c * PLANE + r * PW] = 0.f;
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
                float v = bsum[u];
                v = v + __shfl_xor(v, 8, 64);
                v = v + __shfl_xor(v, 4, 64);
                v = v + __shfl_xor(v, 2, 64);
                v = v + __shfl_xor(v, 1, 64);
                if (gq == 0) p.bpart[(i64)bzi * p.part_stride + oc0 + grow + 16 * u] = v;
            }
        }
    }
    // The WK waves that split the pixel rows hold partial sums of the same outputs, added here through LDS (the stage buffers
    // are free after the loop's last barrier) in order of the segment, so a block leaves one partial sum.
    float* out = p.part + (i64)bzi * p.part_stride;
    const int ldo = KK * p.Cin;
    auto store = [&](int t, int e, float v) __attribute__((always_inline)) {
        const int oc = oc0 + wmo * 32 + igemm::Mfma<float>::row(e, lane);
        out[(i64)oc * ldo + t * p.Cin + c0 + l32] = v;
    };
    if constexpr (WK == 4) {
        // four segments: tap by tap, the first segment's wave adds and stores (measured faster than the scheme below, whose
        // four per-wave code paths are each fetched cold)
        float* red = smem;  // [4 waves][16][64]
#pragma unroll
        for (int t = 0; t < KK; ++t) {
            if (wk != 0) {
#pragma unroll
                for (int e = 0; e < 16; ++e) red[(wave * 16 + e) * 64 + lane] = acc[t][e];
            }
            __syncthreads();
            if (wk == 0) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    float v = acc[t][e];
#pragma unroll
                    for (int q = 1; q < WK; ++q) v = v + red[((wave + q * WMO) * 16 + e) * 64 + lane];
                    store(t, e, v);
                }
            }
            __syncthreads();
        }
    } else if constexpr (WK == 2) {
        // two segments: tap t is finished by the wave of segment t % 2; every wave leaves the taps it does not finish in LDS and
        // after one barrier adds and stores the ones it does, so all four waves share the additions and the stores
        constexpr int NS = S::NS;
        float* red = smem;  // [4 waves][NS][16][64]
#pragma unroll
        for (int k = 0; k < WK; ++k) {
            if (wk != k) continue;  // scalar
#pragma unroll
            for (int t = 0; t < KK; ++t) {
                if (t % WK == k) continue;
#pragma unroll
                for (int e = 0; e < 16; ++e) red[((wave * NS + slot(t, k, WK)) * 16 + e) * 64 + lane] = acc[t][e];
                __builtin_amdgcn_sched_barrier(0);  // tap by tap: the values of one tap in flight, not of all
            }
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < WK; ++k) {
            if (wk != k) continue;
#pragma unroll
            for (int t = 0; t < KK; ++t) {
                if (t % WK != k) continue;
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    float v = 0.f;
#pragma unroll
                    for (int q = 0; q < WK; ++q) {
                        const float term = q == k ? acc[t][e] : red[(((wmo + q * WMO) * NS + slot(t, q, WK)) * 16 + e) * 64 + lane];
                        v = q == 0 ? term : v + term;
                    }
                    store(t, e, v);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    } else {
#pragma unroll
        for (int t = 0; t < KK; ++t)
#pragma unroll
            for (int e = 0; e < 16; ++e) store(t, e, acc[t][e]);
    }
}

struct Plan {
    bool ok = false;
    int WMO = 0, OW = 0, R = 0, splits = 1, sps = 1, stages = 0;
    size_t smem = 0;
};

// Instantiated (WMO, OW, R): rows of 16 and 32 pixels (maps 32 and 64 wide); of 28 pixels (56 wide; a segment of 7 pixels cannot be
// walked in pairs, so no layout with four row segments); of 8 pixels, a whole 8 x 8 output per stage (16 wide).
#define FX_WG2_SHAPES(X) X(1, 16, 4) X(2, 16, 4) X(4, 16, 4) X(1, 32, 2) X(2, 32, 2) X(4, 32, 2) X(2, 28, 2) X(4, 28, 2) X(1, 8, 8) X(2, 8, 8) X(4, 8, 8) X(4, 14, 2)

inline Plan make_plan(int num_cus, i64 B, i64 Cin, i64 H, i64 W, i64 Cout, i64 kh, i64 kw, i64 sh, i64 sw, i64 ph, i64 pw, i64 oh, i64 ow) {
    Plan pl;
    if (kh != 3 || kw != 3 || sh != 2 || sw != 2 || pw != 1 || ph > 1 || W != 2 * ow || Cin % CT != 0 || Cout % 32 != 0) return pl;
    if (Cout * Cin * KK > 0x7fffffff || 32 * H * W * 4 > 0x7fffffff || Cout * oh * ow * 4 > 0x7fffffff) return pl;
    const int wmo = Cout % 128 == 0 ? 4 : Cout % 64 == 0 ? 2 : 1;
#define FX_WG2_PICK(A, O, RR)                                            \
    if (!pl.ok && wmo == A && ow == O && oh % RR == 0) {                 \
        pl.ok = true; pl.WMO = A; pl.OW = O; pl.R = RR;                  \
        pl.smem = Shape<A, O, RR>::LDS;                                  \
    }
    FX_WG2_SHAPES(FX_WG2_PICK)
#undef FX_WG2_PICK
    if (!pl.ok) return pl;
    pl.ok = false;
    pl.stages = (int)(B * (oh / pl.R));
    const i64 tiles = (Cin / CT) * (Cout / (32 * pl.WMO));
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
    return (i64)pl.splits * (Cout * Cin * KK + (with_bias ? Cout : 0)) * (i64)sizeof(float);
}

// x, g and part must be 16-byte aligned.
// act / db non-null: the masked variant (act 16-byte aligned as well).
inline int run(fx_ctx* c, const Plan& pl, const float* x, const float* g, float* dw, float* part, i64 Cin, i64 H, i64 Cout, i64 ph, i64 oh,
               const float* act = nullptr, float* db = nullptr) {
    Params p;
    p.x = x; p.g = g; p.part = part; p.act = act; p.bpart = part + Cout * Cin * KK;
    p.Cin = (int)Cin; p.H = (int)H; p.Cout = (int)Cout; p.oh = (int)oh; p.ph = (int)ph;
    p.stages = pl.stages; p.sps = pl.sps; p.spi = (int)(oh / pl.R);
    p.div_spi = FastDiv((uint32_t)p.spi);
    p.part_stride = Cout * Cin * KK + (act ? Cout : 0);
    const dim3 grid((unsigned)(Cin / CT), (unsigned)(Cout / (32 * pl.WMO)), (unsigned)pl.splits);
    const i64 blocks = (i64)grid.x * grid.y * grid.z;
    p.xcd_chunk = blocks % 8 == 0 && blocks <= 0x7fffffff ? (int)(blocks / 8) : 0;
    bool launched = false;
#define FX_WG2_LAUNCH(A, O, RR)                                                                                        \
    if (!launched && pl.WMO == A && pl.OW == O && pl.R == RR) {                                                        \
        static const hipError_t attr = hipFuncSetAttribute((const void*)wgrad_s2_kernel<A, O, RR, false>,              \
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_LIMIT); \
        static const hipError_t attr_m = hipFuncSetAttribute((const void*)wgrad_s2_kernel<A, O, RR, true>,             \
                                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_LIMIT); \
        FX_HIP_CHECK(attr);                                                                                            \
        FX_HIP_CHECK(attr_m);                                                                                          \
        if (act) FX_LAUNCH(grid, dim3(NT), pl.smem, c->stream, (p), wgrad_s2_kernel<A, O, RR, true>);                           \
        else FX_LAUNCH(grid, dim3(NT), pl.smem, c->stream, (p), wgrad_s2_kernel<A, O, RR, false>);                              \
        launched = true;                                                                                               \
    }
    FX_WG2_SHAPES(FX_WG2_LAUNCH)
#undef FX_WG2_LAUNCH
    FX_REQUIRE(launched, "wgrad stride-2 patch kernel: unexpected shape (%d, %d, %d)", pl.WMO, pl.OW, pl.R);
    FX_LAUNCH_CHECK();
    const int n = (int)(Cout * Cin * KK);
    const wgp::ReduceTail tail{p.part_stride, act ? db : nullptr, act ? (int)Cout : 0};
    const FastDiv div_row((uint32_t)(KK * Cin)), div_cin((uint32_t)Cin);
    // (with the bias sums behind each partial the stride stays a multiple of 4 floats: Cout % 32 == 0)
    if (pl.splits >= 128 && n <= (1 << 17) && n % 4 == 0 && Cin % 4 == 0 && fx::aligned16(part))
        FX_LAUNCH(dim3((unsigned)(fx::ceil_div((i64)n, 64) + wgp::tail_blocks(tail, 16))), dim3(256), 0, c->stream, (part, dw, n, pl.splits, (int)Cin, div_row, div_cin, tail), wgp::wgrad_patch_reduce_vec_kernel<16>);
    else if (pl.splits >= 128 && n <= (1 << 17))
        FX_LAUNCH(dim3((unsigned)(fx::ceil_div((i64)n, 16) + wgp::tail_blocks(tail, 16))), dim3(256), 0, c->stream, (part, dw, n, pl.splits, (int)Cin, div_row, div_cin, tail), wgp::wgrad_patch_reduce_grouped_kernel<16>);
    else
        FX_LAUNCH(dim3((unsigned)(fx::ceil_div((i64)n, 256) + wgp::tail_blocks(tail, 256))), dim3(256), 0, c->stream, (part, dw, n, pl.splits, (int)Cin, div_row, div_cin, tail), wgp::wgrad_patch_reduce_kernel);
    FX_LAUNCH_CHECK();
    return FX_OK;
}

}  // namespace wg2
