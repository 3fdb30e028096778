// Forward pass of a 3x3 convolution of stride 2 and padding 1 over an even-sized map (f64), the twin of fwd_patch_s2.hpp on
// v_mfma_f64_16x16x4_f64:
//   y[b][oc][oy][ox] = bias[oc] + sum over (c, ky, kx) of w[oc][c][ky][kx] * x[b][c][2 oy + ky - 1][2 ox + kx - 1]
// (conv2d_impl, src/backend/storage/extensions/convolutions.rs:218-266).
//
// A block (8 waves) takes 256 output pixels of one image -- TR = 256 / OW output rows -- and MB blocks of 32 output channels; a
// wave owns 32 pixels x all of them as 2 MB x 2 accumulator blocks of 16 (oc) x 16 (pixels).  Input channels are reduced four at
// a time (one MFMA step per tap); per chunk of 4 the block holds
//   Ws[tap][oc block][lane]      the MFMA A operand as the lanes read it: lane l holds w[oc = 16 block + l % 16][c = l / 16][tap]
//                                (read from w in its own layout, no re-layout kernel)
//   Xs[c][row][parity][col / 2]  the 2 TR + 1 patch rows, even and odd patch columns in separate half rows: the pixels of a
//                                wave then read consecutive words for every tap although the layer strides by 2
// in two LDS buffers (next chunk loaded into registers before the MFMA loop of the current one, parked after it, one barrier
// per chunk).  Per tap a wave reads 2 MB weights + 2 patch values for 4 MB MFMAs.  Bias (+ReLU) ride in the store.
#pragma once
#include <cstdlib>

#include "igemm_core.hpp"

namespace fwd2 {
using igemm::FastDiv;
using igemm::f64x4;

constexpr int KK = 9, NT = 512, CC = 4, PIX = 256;
constexpr size_t LDS_LIMIT = 160 * 1024;

struct Params {
    const double* x;
    const double* w;
    double* y;
    const double* bias;  // or null
    int relu;
    int Cin, Cout, H, oh, tpi, nmt;  // tiles per image, oc tiles of 32 MB
    FastDiv div_nmt, div_tpi;
};

__device__ __forceinline__ double2 ldg2(const double* base, uint32_t byteoff) {
    typedef __attribute__((address_space(1))) const char gchar;
    typedef double v2 __attribute__((ext_vector_type(2)));
    typedef __attribute__((address_space(1))) const v2 gv2;
    const v2 v = *(gv2*)((gchar*)base + byteoff);
    return make_double2(v.x, v.y);
}

template <int OW, int MB>
struct Shape {
    static constexpr int TR = PIX / OW, PR = 2 * TR + 1, W = 2 * OW;
    static constexpr int HALF = OW + 1;                       // entries of a parity half row (even: patch columns 0, 2, .., 2 OW)
    static constexpr int RP = OW == 16 ? 40 : 2 * HALF;       // row pitch: two half rows
    static constexpr int PLANE = (PR * RP) | 1;
    static constexpr int NB = 2 * MB;                         // blocks of 16 output channels
    static constexpr int WCH = KK * NB * 64, XCH = CC * PLANE, BUF = WCH + XCH;
    static constexpr size_t LDS = 2 * (size_t)BUF * sizeof(double);
    static constexpr int W2 = MB * 32 * CC * KK / 2;          // double2 of a weight chunk (36 contiguous doubles per oc)
    static constexpr int NWP = (W2 + NT - 1) / NT;
    static constexpr int X2 = CC * PR * (W / 2);              // double2 of a patch chunk
    static constexpr int NXP = (X2 + NT - 1) / NT;
    static_assert(PIX % OW == 0 && OW % 16 == 0 && 2 * HALF <= RP && LDS <= LDS_LIMIT, "shape");
};

template <int OW, int MB, bool BIAS>
__global__ __launch_bounds__(NT, 1) void fwd_s2_f64_kernel(const Params p) {
    using S = Shape<OW, MB>;
    constexpr int TR = S::TR, PR = S::PR, W = S::W, RP = S::RP, PLANE = S::PLANE, WCH = S::WCH, BUF = S::BUF, HALF = S::HALF, NB = S::NB;
    FX_DYNAMIC_SMEM(double, smem_fwd2);
    double* smem = smem_fwd2;
    const int tid = threadIdx.x, lane = tid & 63, kq = lane >> 4, l16 = lane & 15;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int bt = (int)p.div_nmt.div(blockIdx.x), mt = (int)blockIdx.x - bt * p.nmt;
    const int b = (int)p.div_tpi.div((uint32_t)bt), tile = bt - b * p.tpi;
    const int oc0 = mt * 32 * MB, oy0 = tile * TR, iy0 = 2 * oy0 - 1;
    const int L = p.oh * OW;

    // staging maps (constant over the chunks): weight double2 f -> (oc, 18 double2 of its 36 doubles); patch double2 f -> (c, row, 2 columns)
    const double2 zero2 = make_double2(0., 0.);
    double2 wv[S::NWP], xv[S::NXP];
    const double* wsrc = p.w + (i64)oc0 * p.Cin * KK;
    const double* xsrc = p.x + (i64)b * p.Cin * p.H * W;
    auto prefetch = [&](int k) __attribute__((always_inline)) {
        const int c0 = k * CC;
#pragma unroll
        for (int u = 0; u < S::NWP; ++u) {
            const int f = u * NT + tid;
            const bool ok = (u + 1) * NT <= S::W2 || f < S::W2;
            const int ocl = f / 18, q = f - ocl * 18;
            wv[u] = ldg2(wsrc + (i64)c0 * KK, ok ? (uint32_t)(ocl * p.Cin * KK + 2 * q) * 8u : 0u);
        }
#pragma unroll
        for (int u = 0; u < S::NXP; ++u) {
            const int f = u * NT + tid;
            const bool in = (u + 1) * NT <= S::X2 || f < S::X2;
            const int cr = f / (W / 2), q = f - cr * (W / 2), c = cr / PR, r = cr - c * PR;
            const int iy = iy0 + r;
            const bool ok = in && iy >= 0 && iy < p.H;
            xv[u] = ldg2(xsrc + (i64)c0 * p.H * W, ok ? (uint32_t)((c * p.H + iy) * W + 2 * q) * 8u : 0u);
            if (!ok) xv[u] = zero2;
        }
    };
    auto park = [&](int buf) __attribute__((always_inline)) {
        double* Ws = smem + buf * BUF;
        double* Xs = Ws + WCH;
#pragma unroll
        for (int u = 0; u < S::NWP; ++u) {
            const int f = u * NT + tid;
            if ((u + 1) * NT <= S::W2 || f < S::W2) {
                const int ocl = f / 18, q = f - ocl * 18;
                const double v[2] = {wv[u].x, wv[u].y};
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    const int e = 2 * q + i, cl = e / KK, t = e - cl * KK;
                    Ws[(t * NB + (ocl >> 4)) * 64 + cl * 16 + (ocl & 15)] = v[i];
                }
            }
        }
#pragma unroll
        for (int u = 0; u < S::NXP; ++u) {
            const int f = u * NT + tid;
            if ((u + 1) * NT <= S::X2 || f < S::X2) {
                const int cr = f / (W / 2), q = f - cr * (W / 2), c = cr / PR, r = cr - c * PR;
                // input columns 2q, 2q+1 are patch columns 2q+1 (odd, entry q) and 2q+2 (even, entry q+1)
                double* d = Xs + c * PLANE + r * RP + q;
                d[HALF] = xv[u].x;
                d[1] = xv[u].y;
            }
        }
    };

    f64x4 acc[NB][2];  // [block of 16 output channels][pixel half]
#pragma unroll
    for (int m = 0; m < NB; ++m)
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[m][h][e] = 0.;

    // this wave's pixels: wave * 32 + 16 h + l16 of the tile, row-major; lane l reads the patch plane of channel l / 16
    int xb0[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int pix = wave * 32 + 16 * h + l16;
        xb0[h] = WCH + kq * PLANE + 2 * (pix / OW) * RP + pix % OW;
    }
    auto compute = [&](int buf) __attribute__((always_inline)) {
        const double* wa = smem + buf * BUF + lane;
        double a[KK][NB], bq[KK][2];
#pragma unroll
        for (int t = 0; t < KK; ++t) {
            const int ky = t / 3, kx = t % 3;
#pragma unroll
            for (int m = 0; m < NB; ++m) a[t][m] = wa[(t * NB + m) * 64];
            // tap column kx: patch column 2 ox + kx -> even half entry ox (kx = 0), odd half entry ox (kx = 1), even entry ox + 1 (kx = 2)
#pragma unroll
            for (int h = 0; h < 2; ++h) bq[t][h] = smem[buf * BUF + xb0[h] + ky * RP + (kx == 1 ? HALF : 0) + (kx == 2 ? 1 : 0)];
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < KK; ++t)
#pragma unroll
            for (int m = 0; m < NB; ++m)
#pragma unroll
                for (int h = 0; h < 2; ++h) acc[m][h] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[t][m], bq[t][h], acc[m][h], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    };

    const int nchunks = p.Cin / CC;
    prefetch(0);
    // patch column 0 (the even half row's entry 0) is the zero padding left of the map: written once in both buffers
    for (int i = tid; i < 2 * CC * PR; i += NT) {
        const int buf = i / (CC * PR), rem = i - buf * (CC * PR), c = rem / PR, r = rem - c * PR;
        smem[buf * BUF + WCH + c * PLANE + r * RP] = 0.;
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

#pragma unroll
    for (int h = 0; h < 2; ++h) {
        double* out = p.y + ((i64)b * p.Cout + oc0) * L + (i64)oy0 * OW + wave * 32 + 16 * h + l16;
#pragma unroll
        for (int m = 0; m < NB; ++m)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int oc = 16 * m + igemm::Mfma<double>::row(e, lane);
                double v = acc[m][h][e];
                if constexpr (BIAS) {
                    v = v + p.bias[oc0 + oc];
                    if (p.relu) v = v > 0. ? v : 0.;
                }
                out[(i64)oc * L] = v;
            }
    }
}

struct Plan {
    bool ok = false;
    int OW = 0, MB = 0;
    size_t smem = 0;
};

// Instantiated (OW, MB): maps 32 and 64 wide, 32 or 64 output channels per block.
#define FX_FWD2_SHAPES(X) X(16, 2) X(16, 1) X(32, 2) X(32, 1)

inline Plan make_plan(i64 B, i64 Cin, i64 H, i64 W, i64 Cout, i64 kh, i64 kw, i64 sh, i64 sw, i64 ph, i64 pw, i64 oh, i64 ow) {
    Plan pl;
    if (kh != 3 || kw != 3 || sh != 2 || sw != 2 || ph != 1 || pw != 1 || W != 2 * ow || H != 2 * oh || Cin % CC != 0 || Cout % 32 != 0) return pl;
    if (Cin * H * W * 8 > 0x7fffffff || Cout * Cin * KK * 8 > 0x7fffffff || B * oh * (Cout / 32) > 0x7fffffff) return pl;
    // Measured against the implicit GEMM (256 images, 32x32 maps): 54.7 against 62.8 us at 32 -> 64 channels, 28.9 against 43.7 us
    // at 32 -> 32; with two or more blocks of output channels per pixel tile the patch is staged once per block and the
    // implicit GEMM wins (186 against 180 us at 64 -> 128, 366 against 337 us at [128,64,64,64] -> 128).
    if (Cout != 32 && Cout != 64) return pl;
    const int mb = Cout % 64 == 0 ? 2 : 1;
#define FX_FWD2_PICK(O, M_)                                                                  \
    if (!pl.ok && ow == O && mb == M_ && oh % (PIX / O) == 0) {                              \
        pl.ok = true; pl.OW = O; pl.MB = M_; pl.smem = Shape<O, M_>::LDS;                    \
    }
    FX_FWD2_SHAPES(FX_FWD2_PICK)
#undef FX_FWD2_PICK
    return pl;
}

// x, w and y must be 16-byte aligned.
inline int run(fx_ctx* c, const Plan& pl, const double* x, const double* w, double* y, i64 B, i64 Cin, i64 H, i64 Cout, i64 oh, const double* bias,
               int relu) {
    Params p;
    p.x = x; p.w = w; p.y = y; p.bias = bias; p.relu = relu;
    p.Cin = (int)Cin; p.Cout = (int)Cout; p.H = (int)H; p.oh = (int)oh;
    p.tpi = (int)(oh / (PIX / pl.OW));
    p.nmt = (int)(Cout / (32 * pl.MB));
    p.div_nmt = FastDiv((uint32_t)p.nmt);
    p.div_tpi = FastDiv((uint32_t)p.tpi);
    const dim3 grid((unsigned)(B * p.tpi * p.nmt));
    bool launched = false;
#define FX_FWD2_LAUNCH(O, M_)                                                                                          \
    if (!launched && pl.OW == O && pl.MB == M_) {                                                                      \
        static const hipError_t attr0 = hipFuncSetAttribute((const void*)fwd_s2_f64_kernel<O, M_, false>,              \
                                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_LIMIT); \
        static const hipError_t attr1 = hipFuncSetAttribute((const void*)fwd_s2_f64_kernel<O, M_, true>,               \
                                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_LIMIT); \
        FX_HIP_CHECK(attr0);                                                                                           \
        FX_HIP_CHECK(attr1);                                                                                           \
        if (bias) FX_LAUNCH(grid, dim3(NT), pl.smem, c->stream, (p), fwd_s2_f64_kernel<O, M_, true>);                           \
        else FX_LAUNCH(grid, dim3(NT), pl.smem, c->stream, (p), fwd_s2_f64_kernel<O, M_, false>);                               \
        launched = true;                                                                                               \
    }
    FX_FWD2_SHAPES(FX_FWD2_LAUNCH)
#undef FX_FWD2_LAUNCH
    FX_REQUIRE(launched, "fwd stride-2 patch kernel (f64): unexpected shape (%d, %d)", pl.OW, pl.MB);
    FX_LAUNCH_CHECK();
    return FX_OK;
}

}  // namespace fwd2
