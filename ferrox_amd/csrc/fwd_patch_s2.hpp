// Forward pass of a 3x3 convolution of stride 2 and padding 1 over an even-sized map (f32):
//   y[b][oc][oy][ox] = bias[oc] + sum over (c, ky, kx) of w[oc][c][ky][kx] * x[b][c][2 oy + ky - 1][2 ox + kx - 1]
// (conv2d_impl, src/backend/storage/extensions/convolutions.rs:218-266), the forward member of the stride-2 family of
// dgrad_patch_s2.hpp / wgrad_patch_s2.hpp.
//
// The stride-1 patch kernel serves such a layer through a tall-patch instantiation plus a weight-image kernel; for layers of
// few channels that second launch and the tall patch's idle rows are a third of the time.  Here a block
// (8 waves) takes 256 output pixels of one image -- TR = 256 / OW output rows -- and MB blocks of 32 output channels; a wave
// owns 32 pixels x all of them (MB accumulator blocks).  Input channels are reduced in chunks of 8; per chunk the block holds
//   Ws[c pair][tap][oc block][lane]   the MFMA A operand as the lanes read it: lane l holds w[oc = 32 block + l % 32][c = 2 pair + l / 32][tap]
//                                     (read from w in its own layout, no re-layout kernel)
//   Xs[c][row][parity][col / 2]       the 2 TR + 1 patch rows, even and odd patch columns in separate half rows: the pixels of
//                                     a wave then read consecutive words for every tap although the layer strides by 2
// in two LDS buffers (next chunk loaded into registers before the MFMA loop of the current one, parked after it, one barrier
// per chunk).  Per channel pair a wave reads 9 patch values + 9 MB weights for 9 MB MFMAs.  Bias (+ReLU) ride in the store.
#pragma once
#include <cstdlib>

#include "igemm_core.hpp"

namespace fw2 {
using igemm::FastDiv;
using igemm::f32x16;
using igemm::ldg4;

constexpr int KK = 9, NT = 512, CC = 8, PIX = 256;
constexpr size_t LDS_LIMIT = 160 * 1024;

struct Params {
    const float* x;
    const float* w;
    float* y;
    const float* bias;  // or null
    int relu;
    int Cin, Cout, H, oh, tpi, nmt;  // tiles per image, oc tiles of 32 MB
    FastDiv div_nmt, div_tpi;
};

template <int OW, int MB>
struct Shape {
    static constexpr int TR = PIX / OW, PR = 2 * TR + 1, W = 2 * OW;
    static constexpr int HALF = OW + 1;                       // entries of a parity half row (even: patch columns 0, 2, .., 2 OW)
    // row pitch: two half rows, padded so that two output rows down (4 patch rows... 2 RP words) lands 16 banks further when a
    // wave's 32 pixels span two output rows (OW = 16)
    static constexpr int RP = OW == 16 ? 40 : 2 * HALF;
    static constexpr int PLANE = (PR * RP) | 1;
    static constexpr int WCH = (CC / 2) * KK * MB * 64, XCH = CC * PLANE, BUF = WCH + XCH;
    static constexpr size_t LDS = 2 * (size_t)BUF * sizeof(float);
    static constexpr int W4 = MB * 32 * CC * KK / 4;          // float4 of a weight chunk (72 contiguous floats per oc)
    static constexpr int NWP = (W4 + NT - 1) / NT;
    static constexpr int X4 = CC * PR * (W / 4);              // float4 of a patch chunk
    static constexpr int NXP = (X4 + NT - 1) / NT;
    static_assert(PIX % OW == 0 && OW % 4 == 0 && 2 * HALF <= RP && LDS <= LDS_LIMIT, "shape");
};

template <int OW, int MB, bool BIAS>
__global__ __launch_bounds__(NT, 1) void fwd_s2_kernel(const Params p) {
    using S = Shape<OW, MB>;
    constexpr int TR = S::TR, PR = S::PR, W = S::W, RP = S::RP, PLANE = S::PLANE, WCH = S::WCH, BUF = S::BUF, HALF = S::HALF;
    FX_DYNAMIC_SMEM(float, smem);
    const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5, l32 = lane & 31;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int bt = (int)p.div_nmt.div(blockIdx.x), mt = (int)blockIdx.x - bt * p.nmt;
    const int b = (int)p.div_tpi.div((uint32_t)bt), tile = bt - b * p.tpi;
    const int oc0 = mt * 32 * MB, oy0 = tile * TR, iy0 = 2 * oy0 - 1;
    const int L = p.oh * OW;

    // staging maps (constant over the chunks): weight float4 f -> (oc, 18 float4 of its 72 floats); patch float4 f -> (c, row, 4 columns)
    const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
    float4 wv[S::NWP], xv[S::NXP];
    const float* wsrc = p.w + (i64)oc0 * p.Cin * KK;
    const float* xsrc = p.x + (i64)b * p.Cin * p.H * W;
    auto prefetch = [&](int k) __attribute__((always_inline)) {
        const int c0 = k * CC;
#pragma unroll
        for (int u = 0; u < S::NWP; ++u) {
            const int f = u * NT + tid;
            const bool ok = (u + 1) * NT <= S::W4 || f < S::W4;
            const int ocl = f / 18, q = f - ocl * 18;
            wv[u] = ldg4(wsrc + (i64)c0 * KK, ok ? (uint32_t)(ocl * p.Cin * KK + 4 * q) * 4u : 0u);
        }
#pragma unroll
        for (int u = 0; u < S::NXP; ++u) {
            const int f = u * NT + tid;
            const bool in = (u + 1) * NT <= S::X4 || f < S::X4;
            const int cr = f / (W / 4), q = f - cr * (W / 4), c = cr / PR, r = cr - c * PR;
            const int iy = iy0 + r;
            const bool ok = in && iy >= 0 && iy < p.H;
            xv[u] = ldg4(xsrc + (i64)c0 * p.H * W, ok ? (uint32_t)((c * p.H + iy) * W + 4 * q) * 4u : 0u);
            if (!ok) xv[u] = zero4;
        }
    };
    auto park = [&](int buf) __attribute__((always_inline)) {
        float* Ws = smem + buf * BUF;
        float* Xs = Ws + WCH;
#pragma unroll
        for (int u = 0; u < S::NWP; ++u) {
            const int f = u * NT + tid;
            if ((u + 1) * NT <= S::W4 || f < S::W4) {
                const int ocl = f / 18, q = f - ocl * 18;
                const float v[4] = {wv[u].x, wv[u].y, wv[u].z, wv[u].w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int e = 4 * q + i, cl = e / KK, t = e - cl * KK;
                    Ws[(((cl >> 1) * KK + t) * MB + (ocl >> 5)) * 64 + (cl & 1) * 32 + (ocl & 31)] = v[i];
                }
            }
        }
#pragma unroll
        for (int u = 0; u < S::NXP; ++u) {
            const int f = u * NT + tid;
            if ((u + 1) * NT <= S::X4 || f < S::X4) {
                const int cr = f / (W / 4), q = f - cr * (W / 4), c = cr / PR, r = cr - c * PR;
                // input columns 4q .. 4q+3 are patch columns 4q+1 .. 4q+4: odd, even, odd, even
                float* d = Xs + c * PLANE + r * RP + 2 * q;
                d[HALF] = xv[u].x;      // odd  (4q + 1) / 2 = 2q
                d[1] = xv[u].y;         // even (4q + 2) / 2 = 2q + 1
                d[HALF + 1] = xv[u].z;  // odd  2q + 1
                d[2] = xv[u].w;         // even 2q + 2
            }
        }
    };

    f32x16 acc[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[m][e] = 0.f;

    // this wave's pixels: wave * 32 + l32 of the tile, row-major; lane l reads the patch plane of c = 2 pair + l / 32
    const int pix = wave * 32 + l32, prow = pix / OW, pcol = pix % OW;
    const int xb0 = WCH + half * PLANE + 2 * prow * RP + pcol;
    auto compute = [&](int buf) __attribute__((always_inline)) {
        const float* wa = smem + buf * BUF + lane;
        const float* xb = smem + buf * BUF + xb0;
        float a[CC / 2][KK][MB], bq[CC / 2][KK];
        auto rd = [&](int cp) __attribute__((always_inline)) {
#pragma unroll
            for (int t = 0; t < KK; ++t) {
                const int ky = t / 3, kx = t % 3;
#pragma unroll
                for (int m = 0; m < MB; ++m) a[cp][t][m] = wa[((cp * KK + t) * MB + m) * 64];
                // tap column kx: patch column 2 ox + kx -> even half entry ox (kx = 0), odd half entry ox (kx = 1), even entry ox + 1 (kx = 2)
                bq[cp][t] = xb[2 * cp * PLANE + ky * RP + (kx == 1 ? HALF : 0) + (kx == 2 ? 1 : 0)];
            }
            __builtin_amdgcn_sched_barrier(0);
        };
        rd(0);
#pragma unroll
        for (int cp = 0; cp < CC / 2; ++cp) {
            if (cp + 1 < CC / 2) rd(cp + 1);
#pragma unroll
            for (int t = 0; t < KK; ++t)
#pragma unroll
                for (int m = 0; m < MB; ++m) acc[m] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[cp][t][m], bq[cp][t], acc[m], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    const int nchunks = p.Cin / CC;
    prefetch(0);
    // patch column 0 (the even half row's entry 0) is the zero padding left of the map: written once in both buffers
    for (int i = tid; i < 2 * CC * PR; i += NT) {
        const int buf = i / (CC * PR), rem = i - buf * (CC * PR), c = rem / PR, r = rem - c * PR;
        smem[buf * BUF + WCH + c * PLANE + r * RP] = 0.f;
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

    float* out = p.y + ((i64)b * p.Cout + oc0) * L + (i64)oy0 * OW + pix;
#pragma unroll
    for (int m = 0; m < MB; ++m)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const int oc = m * 32 + igemm::Mfma<float>::row(e, lane);
            float v = acc[m][e];
            if constexpr (BIAS) {
                v = v + p.bias[oc0 + oc];
                if (p.relu) v = v > 0.f ? v : 0.f;
            }
            out[(i64)oc * L] = v;
        }
}

struct Plan {
    bool ok = false;
    int OW = 0, MB = 0;
    size_t smem = 0;
};

// Instantiated (OW, MB): maps 32 and 64 wide, 32 or 64 output channels per block.
#define FX_FW2_SHAPES(X) X(16, 2) X(16, 1) X(32, 2) X(32, 1)

inline Plan make_plan(i64 B, i64 Cin, i64 H, i64 W, i64 Cout, i64 kh, i64 kw, i64 sh, i64 sw, i64 ph, i64 pw, i64 oh, i64 ow) {
    Plan pl;
    if (kh != 3 || kw != 3 || sh != 2 || sw != 2 || ph != 1 || pw != 1 || W != 2 * ow || H != 2 * oh || Cin % CC != 0 || Cout % 32 != 0) return pl;
    if (Cin * H * W * 4 > 0x7fffffff || Cout * Cin * KK * 4 > 0x7fffffff || B * oh * (Cout / 32) > 0x7fffffff) return pl;
    // Measured against the tall-patch instantiation of the stride-1 kernel (256 images, 32x32 maps): 20.5 against 30.0 us at
    // 32 -> 32 channels, 7.4 against 12.3 us at 8 -> 32, 11.3 against 13.5 us at 8 -> 64, level at 16 -> 64 and 32 -> 64, and
    // slower from there on (59.6 against 49.6 us at 32 -> 96, 199 against 153 us at [128,64,64,64] -> 128): this kernel takes
    // the layers whose output channels fit one block and whose reduction is short.
    if (!(Cout == 32 || (Cout == 64 && Cin <= 16))) return pl;
    const int mb = Cout % 64 == 0 ? 2 : 1;
#define FX_FW2_PICK(O, M_)                                                                   \
    if (!pl.ok && ow == O && mb == M_ && oh % (PIX / O) == 0) {                              \
        pl.ok = true; pl.OW = O; pl.MB = M_; pl.smem = Shape<O, M_>::LDS;                    \
    }
    FX_FW2_SHAPES(FX_FW2_PICK)
#undef FX_FW2_PICK
    return pl;
}

// x, w and y must be 16-byte aligned.
inline int run(fx_ctx* c, const Plan& pl, const float* x, const float* w, float* y, i64 B, i64 Cin, i64 H, i64 Cout, i64 oh, const float* bias,
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
#define FX_FW2_LAUNCH(O, M_)                                                                                           \
    if (!launched && pl.OW == O && pl.MB == M_) {                                                                      \
        static const hipError_t attr0 = hipFuncSetAttribute((const void*)fwd_s2_kernel<O, M_, false>,                  \
                                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_LIMIT); \
        static const hipError_t attr1 = hipFuncSetAttribute((const void*)fwd_s2_kernel<O, M_, true>,                   \
                                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_LIMIT); \
        FX_HIP_CHECK(attr0);                                                                                           \
        FX_HIP_CHECK(attr1);                                                                                           \
        if (bias) FX_LAUNCH(grid, dim3(NT), pl.smem, c->stream, (p), fwd_s2_kernel<O, M_, true>);                               \
        else FX_LAUNCH(grid, dim3(NT), pl.smem, c->stream, (p), fwd_s2_kernel<O, M_, false>);                                   \
        launched = true;                                                                                               \
    }
    FX_FW2_SHAPES(FX_FW2_LAUNCH)
#undef FX_FW2_LAUNCH
    FX_REQUIRE(launched, "fwd stride-2 patch kernel: unexpected shape (%d, %d)", pl.OW, pl.MB);
    FX_LAUNCH_CHECK();
    return FX_OK;
}

}  // namespace fw2
