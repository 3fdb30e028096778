// 3x3 convolution forward (f32) with the input patch and the weights staged in LDS; the stride-1 data gradient
// runs through the same kernel as a forward pass over grad_out with flipped, transposed weights.
//
// y[b][m][oy][ox] = sum over (c, ky, kx) of wgt[m][c][ky][kx] * in[b][c][oy*sh+ky-ph][ox*sw+kx-pw]
// (the product the reference forms as filter_2d . im2col(x), src/backend/storage/extensions/convolutions.rs:218-290).
//
// A block (4 waves, WM = 4, 2 or 1 along the output channels) owns BM = 32*WM output channels x 32*TN*(4/WM) consecutive
// output pixels of one image and walks the input channels in chunks of 8 (one stage each).  Per stage it holds in LDS
//   Ws[m][tap*8 + c]   the weights of the chunk, pitch 73 (odd: the 32 lanes of an A read hit 32 banks)
//   Xs[c][row][col]    the zero-padded input rows under the pixel tile, plane pitch odd for the same reason
// so each of the nine taps reads the same patch at a shifted address and no im2col index arithmetic or bounds
// test is left in the MFMA loop.  Ws arrives as a ready-made image (built once per call by wimg_kernel), so its
// staging is a straight 16-byte copy; the patch rows use the regular thread-to-row map of the weight-gradient
// kernel.  The next stage's global loads are issued before the MFMA loop of the current one.
// Rows of up to 64 floats; the persistent variant further down also takes rows of up to 256 (its WIDE staging maps).
#pragma once
#include <array>
#include <cstdio>
#include <cstdlib>

#include "wgrad_patch.hpp"

namespace cpk {
using igemm::FastDiv;
using igemm::f32x16;
using wgp::ldg4;

constexpr int CC = 8, NT = 256, KK = 9;
constexpr int WPITCH = KK * CC + 1;         // 73
constexpr int NXP_SHORT = 4, NXP_TALL = 10;  // patch rows are staged two per pass: up to 8 rows, or 20 (strided layers)
constexpr int NXP_PERSIST = 5;              // persistent variant: up to 10 patch rows
constexpr int NXP_WIDE = 6, NXP_WIDE2 = 8;  // persistent variant, rows of 65 to 128 floats: up to 6 patch rows; 129 to 256: 8 passes = 4 rows
constexpr int LPR = 16;                     // lanes per patch row: W <= 64 (the persistent variant also takes 32: W <= 128)
constexpr int SLACK = 16;
constexpr size_t LDS_BUDGET = 72 * 1024;
// persistent variant: fixed plane pitch (1 mod 4) and buffer size, so that buffer, channel pair and tap column are all
// part of the 16-bit immediate offset of an LDS read: 2 x (8 x 1149 + 16) x 4 bytes = 73664 <= LDS_BUDGET
constexpr int PPLANE = 1149, PBUF = CC * PPLANE + SLACK;
constexpr size_t PP_LDS = 2 * (size_t)PBUF * sizeof(float);
static_assert(PP_LDS <= LDS_BUDGET && (PBUF + 6 * PPLANE + 2) * 4 < 65536 && PPLANE % 4 == 1, "persistent patch buffers");

struct Params {
    const float* x;
    const float* wimg;
    float* y;
    const float* bias;  // optional, per output channel; with relu != 0 the sum is clamped at 0 afterwards
    int relu;
    int C, H, W, M, OH, OW, sh, sw, ph, pw;
    int PR, PW, PLANE, L, tpi, nchunks;
    int xcd_chunk;  // gridDim.x / 8 when that divides: workgroup ids go to the 8 XCDs round-robin, see the kernel
    FastDiv div_tpi, div_ow;
    // small maps (MULTI): a tile holds nimg whole images, image i in patch rows [i * RPI, (i + 1) * RPI)
    int nimg, RPI, B;
    FastDiv div_L, div_rpi;
    // persistent variant: all tiles (mtiles x B x tpi), floats per patch buffer, B * tpi
    int ntiles, bufsz, bt;
    FastDiv div_bt;
};

// Weight images: out[mt][ch][m][tap*8 + cc], zero in column 72 and in rows past the last output channel.
//   flip == 0 (forward):        wgt[m][c][tap]   = w[oc = m][c][tap]
//   flip == 1 (data gradient):  wgt[m][c][tap]   = w[oc = c][cin = m][8 - tap]
__global__ __launch_bounds__(256) void wimg_kernel(const float* __restrict__ w, float* __restrict__ out, int Cout, int Cin, int M,
                                                   int BM, int nchunks, int flip, i64 n) {
    const i64 i = (i64)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const int col = (int)(i % WPITCH);
    i64 r = i / WPITCH;
    const int m = (int)(r % BM);
    r /= BM;
    const int ch = (int)(r % nchunks), mt = (int)(r / nchunks);
    const int mm = mt * BM + m;
    float v = 0.f;
    if (col < KK * CC && mm < M) {
        const int t = col / CC, c = ch * CC + col % CC;
        v = flip ? w[((i64)c * Cin + mm) * KK + (KK - 1 - t)] : w[((i64)mm * Cin + c) * KK + t];
    }
    out[i] = v;
}

// MULTI: maps of at most 64 pixels.  A tile is then nimg whole images stacked in the patch, each with its own zero
// rows above and below, so that the 128 pixels of the smallest tile are not mostly padding.
// NARROW: rows of at most 32 floats are staged by 8 lanes each, four patch rows per pass instead of two (strided layers over
// narrow maps need more patch rows than pixels' worth: a 128-pixel tile of a 14-wide output at stride 2 sits on 23 rows).
template <int WM, int TN, bool BIAS, int NXP, bool MULTI = false, bool NARROW = false>
__global__ __launch_bounds__(NT, 2) void conv_patch_kernel(const Params p) {
    constexpr int BM = 32 * WM, WN = 4 / WM, NPIX = 32 * TN * WN;
    constexpr int LPRN = NARROW ? LPR / 2 : LPR, RPP = NT / (LPRN * CC);  // lanes per patch row, rows per pass
    constexpr int WIMG = BM * WPITCH;             // floats in one weight image
    constexpr int NW = (WIMG / 4 + NT - 1) / NT;  // float4 of the image per thread (the last one only partly used)
    FX_DYNAMIC_SMEM(float, smem);
    float* Ws = smem;
    float* Xs = smem + WIMG;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, l32 = lane & 31;
    // XCD x takes the contiguous range [x * chunk, (x+1) * chunk) of (image, pixel tile) pairs, so neighbouring tiles
    // of an image (which share input rows) and the weight images meet in one L2
    int bx = blockIdx.x;
    if (p.xcd_chunk) bx = (bx & 7) * p.xcd_chunk + (bx >> 3);
    const int b = MULTI ? bx * p.nimg : (int)p.div_tpi.div((uint32_t)bx);  // (first) image of the tile
    const int wm = wave % WM, wn = wave / WM;
    const int pix0 = MULTI ? 0 : (bx - b * p.tpi) * NPIX;
    const int wpix0 = pix0 + wn * 32 * TN;  // first pixel of this wave's columns
    const int m0 = blockIdx.y * BM;
    const int py0 = (int)p.div_ow.div((uint32_t)pix0);
    const int iy_base = py0 * p.sh - p.ph;

    for (int i = tid; i < CC * p.PLANE + SLACK; i += NT) Xs[i] = 0.f;  // the padding columns stay zero from here on
    int boff[TN];  // LDS offset of this lane's pixel in acc block j (plus the plane of its channel of the pair)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int pi = wpix0 + j * 32 + l32;
        if constexpr (MULTI) {
            const int img = (int)p.div_L.div((uint32_t)pi), rem = pi - img * p.L;
            const int py = (int)p.div_ow.div((uint32_t)rem), px = rem - py * p.OW;
            const bool valid = img < p.nimg && b + img < p.B;
            boff[j] = (valid ? (img * p.RPI + py * p.sh) * p.PW + px * p.sw : 0) + half * p.PLANE;
        } else {
            const int py = (int)p.div_ow.div((uint32_t)pi), px = pi - py * p.OW;
            boff[j] = (pi < p.L ? (py - py0) * p.sh * p.PW + px * p.sw : 0) + half * p.PLANE;
        }
    }
    f32x16 acc[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[j][e] = 0.f;
    __syncthreads();

    // staging: thread t copies float4 t + 256u of the weight image and owns float4 column t % 16 of patch rows
    // 2u + rp of channel (t / 16) % 8, where rp = t / 128 is uniform over a wave (NARROW: column t % 8 of rows 4u + rp,
    // channel (t / 8) % 8, rp = t / 64).
    const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
    const int pq = tid & (LPRN - 1), xc = (tid / LPRN) & (CC - 1), rp = tid / (LPRN * CC);
    // A row of W floats is covered by ceil(W / 4) vectors; the last one is moved back to end at the row's end (it then
    // overlaps its neighbour, which parks the same values), so no load crosses into the next row or past the tensor.
    const bool x_lane = pq < ((p.W + 3) >> 2);
    const int xcol = min(4 * pq, p.W - 4);
    const uint32_t x_off = x_lane ? (uint32_t)(xc * p.H * p.W + xcol) * 4u : 0u;
    const int x_dst0 = WIMG + xc * p.PLANE + p.pw + xcol;
    const float* const wsrc0 = p.wimg + (i64)blockIdx.y * p.nchunks * WIMG;
    const float* const xsrc0 = p.x + (i64)b * p.C * p.H * p.W;
    float4 wv[NW], xv[NXP];
    auto prefetch = [&](int ch) {
        const float* wsrc = wsrc0 + (i64)ch * WIMG;
#pragma unroll
        for (int u = 0; u < NW; ++u) {
            const int idx = tid + u * NT;
            wv[u] = ldg4(wsrc, (uint32_t)((u + 1) * NT <= WIMG / 4 || idx < WIMG / 4 ? idx : 0) * 16u);
        }
        const float* xsrc = xsrc0 + (i64)ch * CC * p.H * p.W;
#pragma unroll
        for (int u = 0; u < NXP; ++u) {
            const int r = RPP * u + rp;
            if constexpr (MULTI) {
                const int img = (int)p.div_rpi.div((uint32_t)r), iy = r - img * p.RPI - p.ph;
                if (r < p.PR && iy >= 0 && iy < p.H && b + img < p.B) xv[u] = ldg4(xsrc + ((i64)img * p.C * p.H + iy) * p.W, x_off);
                else xv[u] = zero4;
            } else {
                const int iy = iy_base + r;
                if (r < p.PR && iy >= 0 && iy < p.H) xv[u] = ldg4(xsrc + (i64)iy * p.W, x_off);  // wave-uniform test
                else xv[u] = zero4;
            }
        }
    };
    auto park = [&]() {
        int xd = x_dst0, wd = tid;
        FX_PIN_VGPR2(xd, wd);  // recompute the addresses here instead of keeping them alive
#pragma unroll
        for (int u = 0; u < NW; ++u) {
            const int idx = wd + u * NT;
            if ((u + 1) * NT <= WIMG / 4 || idx < WIMG / 4) *reinterpret_cast<float4*>(Ws + 4 * idx) = wv[u];
        }
        if (x_lane) {
#pragma unroll
            for (int u = 0; u < NXP; ++u) {
                const int r = RPP * u + rp;
                if (r < p.PR) {  // wave-uniform
                    const float4 v = xv[u];
                    float* d = smem + xd + r * p.PW;
                    d[0] = v.x; d[1] = v.y; d[2] = v.z; d[3] = v.w;
                }
            }
        }
    };

    // One stage: 9 taps x 4 channel pairs, fully unrolled; two register sets alternate so that the LDS reads of
    // step i+1 are in flight while the MFMAs of step i run.
    const float* const wa = Ws + (wm * 32 + l32) * WPITCH + half;
    auto compute = [&]() {
        float a0, b0[TN], a1, b1[TN];
        const float* xrow[3] = {Xs, Xs + p.PW, Xs + 2 * p.PW};
#pragma unroll
        for (int j = 0; j < TN; ++j) FX_PIN_VGPR(boff[j]);  // form the 12 x TN read addresses per stage, not once
        auto rd = [&](float& a, float (&bv)[TN], int step) {
            const int t = step >> 2, cp = step & 3, ky = t / 3, kx = t % 3;
            a = wa[t * CC + 2 * cp];
            const float* src = xrow[ky] + 2 * cp * p.PLANE + kx;
#pragma unroll
            for (int j = 0; j < TN; ++j) bv[j] = src[boff[j]];
            __builtin_amdgcn_sched_barrier(0);
        };
        auto mma = [&](float a, const float (&bv)[TN]) {
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, bv[j], acc[j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        };
        rd(a0, b0, 0);
#pragma unroll
        for (int step = 0; step < KK * 4; step += 2) {
            rd(a1, b1, step + 1);
            mma(a0, b0);
            if (step + 2 < KK * 4) rd(a0, b0, step + 2);
            mma(a1, b1);
        }
    };

    prefetch(0);
    park();
    __syncthreads();
    for (int ch = 0; ch < p.nchunks; ++ch) {
        const bool more = ch + 1 < p.nchunks;
        if (more) prefetch(ch + 1);
        __builtin_amdgcn_s_setprio(3);  // a co-resident block that is staging must not delay these MFMAs
        compute();
        __builtin_amdgcn_s_setprio(0);
        __syncthreads();
        if (more) park();
        __syncthreads();
    }

    float* out = p.y + (i64)b * p.M * p.L;
    float bv[16];  // bias of the 16 output channels this lane stores: 16 independent loads (row clamped, no branches)
#pragma unroll
    for (int e = 0; e < 16; ++e) {
        const int m = m0 + wm * 32 + igemm::Mfma<float>::row(e, lane);
        bv[e] = BIAS ? p.bias[m < p.M ? m : p.M - 1] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        int pi = wpix0 + j * 32 + l32;
        bool valid = pi < p.L;
        float* oj = out;
        if constexpr (MULTI) {
            const int img = (int)p.div_L.div((uint32_t)pi);
            valid = img < p.nimg && b + img < p.B;
            pi -= img * p.L;
            oj = out + (i64)(valid ? img : 0) * p.M * p.L;
        }
        if (valid) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int m = m0 + wm * 32 + igemm::Mfma<float>::row(e, lane);
                if (m < p.M) {
                    float v = acc[j][e];
                    if (BIAS) {
                        v = v + bv[e];
                        if (p.relu) v = v > 0.f ? v : 0.f;
                    }
                    oj[(i64)m * p.L + pi] = v;
                }
            }
        }
    }
}


// ---- persistent variant ------------------------------------------------------------------------------------------
// The kernel above pays, per stage, for parking a 37 KB weight image in LDS between two barriers and, per tile, for a
// prologue (first loads exposed) and an epilogue (a block's slot waits for its stores): measured on the 128 x 64 x 56 x 56 -> 128
// layer, 6.5 % of the time goes to staging and 4 % to the stores.  This variant removes both:
//   * the weights never touch LDS: every lane loads the 36 A values of its output-channel row for a stage as nine 16-byte
//     global loads from an image laid out in MFMA operand order ([32-row block][chunk][tap][lane][channel pair]), one stage
//     ahead, into one of two register sets;
//   * the patch is double-buffered in LDS, so a stage has ONE barrier and the next patch is written while other waves still
//     compute; its row pitch is padded so that the 32 pixels of an MFMA operand read fall on 32 different banks also when
//     the run wraps to the next output row (pitch - OW = 32);
//   * blocks are persistent (two per CU) and walk their tiles with the stage pipeline running across tile boundaries: the
//     loads for a tile's first stage are issued during the previous tile's last stage, and the stores of a finished tile
//     drain while the next one computes;
//   * nothing in the MFMA loop but MFMAs, LDS reads and their waits: plane pitch and buffer size are constants, so buffer,
//     channel pair and filter column ride in the 16-bit offset field of a read (no address add per read), and what derives
//     from the wave index (row tests, row pointers, store bases) is kept in scalar registers.
// Measured on that layer (MI355X, 2.4 GHz): 0.450 ms forward and 0.446 ms data gradient against 0.475 / 0.479 ms for the
// kernel above.  What was tried on top and lost: one block of eight waves per CU with the two halves half a stage out of step
// (s_setprio does not order two waves' MFMAs, the extra barriers cost more than the parking they hide); one wave per SIMD
// with 512 registers, accumulators in AGPRs and tiles of up to 128 x 320; the same with loads, parking and stores dropped
// one by one between the MFMAs instead of between the stages (the interleaved read-wait-MFMA stream itself runs at 82
// cycles per MFMA where five reads followed by five MFMAs run at 70).
// Weight images: out[mb][ch][tap][lane][e] = wgt[m = mb*32 + lane%32][c = ch*8 + 2e + lane/32][tap], zero in rows past M
// (wgt as for wimg_kernel: the filter, or the flipped transposed filter of the data gradient).
__global__ __launch_bounds__(256) void wimg2_kernel(const float* __restrict__ w, float* __restrict__ out, int Cout, int Cin, int M,
                                                    int nchunks, int flip, i64 n) {
    const i64 i = (i64)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const int e = (int)(i & 3), lane = (int)((i >> 2) & 63);
    i64 r = i >> 8;
    const int t = (int)(r % KK);
    r /= KK;
    const int ch = (int)(r % nchunks), mb = (int)(r / nchunks);
    const int mm = mb * 32 + (lane & 31), c = ch * CC + 2 * e + (lane >> 5);
    float v = 0.f;
    if (mm < M) v = flip ? w[((i64)c * Cin + mm) * KK + (KK - 1 - t)] : w[((i64)mm * Cin + c) * KK + t];
    out[i] = v;
}

__device__ __forceinline__ float f4sel(const float4& v, int e) { return e == 0 ? v.x : e == 1 ? v.y : e == 2 ? v.z : v.w; }

// WIDE 1: rows of 65 to 128 floats.  A staging pass is then one patch row of the 8 channels (32 lanes per row) instead of two
// (16 lanes per row), up to NXP_WIDE rows.  WIDE 2: rows of 129 to 256 floats, 64 lanes per row: a pass is one patch row of four
// channels (a wave each), two passes per row, up to 4 rows.  Nothing else differs.
template <int WM, int TN, bool BIAS, int WIDE = 0>
__global__ __launch_bounds__(NT, 2) void conv_patch_persist_kernel(const Params p) {
    constexpr int BM = 32 * WM, WN = 4 / WM, NPIX = 32 * TN * WN, NXP = WIDE == 2 ? NXP_WIDE2 : WIDE ? NXP_WIDE : NXP_PERSIST;
    constexpr int LPRK = LPR << WIDE;  // lanes per patch row
    constexpr int AIMG = KK * 64 * 4;  // floats of one (32-row block, chunk) weight image
    FX_DYNAMIC_SMEM(float, smem);
    const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5, l32 = lane & 31;
    // in a scalar register: what derives from the wave index (rows, pointers, tests) stays on the scalar unit
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WM, wn = wave / WM;
    // this block's tiles: XCD x (workgroup ids go to the 8 XCDs round-robin) owns the contiguous range [x*chunk, (x+1)*chunk)
    // and deals it to its blocks, so neighbouring tiles of an image are in flight together behind one L2
    int q, qstep, qend;
    if (p.xcd_chunk) {
        const int x = blockIdx.x & 7;
        q = x * p.xcd_chunk + (blockIdx.x >> 3);
        qstep = gridDim.x >> 3;
        qend = (x + 1) * p.xcd_chunk;
    } else {
        q = blockIdx.x;
        qstep = gridDim.x;
        qend = p.ntiles;
    }
    if (q >= qend) return;
    for (int i = tid; i < 2 * PBUF; i += NT) smem[i] = 0.f;  // the padding columns of both buffers stay zero from here on

    // geometry of a tile
    int b, m0, pix0, iy_base, py0, mb;
    auto geo = [&](int qq) __attribute__((always_inline)) {
        const int mt = (int)p.div_bt.div((uint32_t)qq), rem = qq - mt * p.bt;
        b = (int)p.div_tpi.div((uint32_t)rem);
        pix0 = (rem - b * p.tpi) * NPIX;
        py0 = (int)p.div_ow.div((uint32_t)pix0);
        iy_base = py0 * p.sh - p.ph;
        m0 = mt * BM;
        mb = mt * WM + wm;
    };
    // byte offsets into a patch buffer of this lane's B operands, one set per filter row: everything else about a read
    // (buffer, channel pair, filter column) is a compile-time constant and rides in the instruction's offset field
    int boff[3][TN];
    auto set_boff = [&]() __attribute__((always_inline)) {
        const int wpix0 = pix0 + wn * 32 * TN;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int pi = wpix0 + j * 32 + l32;
            const int py = (int)p.div_ow.div((uint32_t)pi), px = pi - py * p.OW;
            const int o = (pi < p.L ? (py - py0) * p.sh * p.PW + px * p.sw : 0) + half * PPLANE;
#pragma unroll
            for (int ky = 0; ky < 3; ++ky) boff[ky][j] = (o + ky * p.PW) * 4;
        }
    };
    f32x16 acc[TN];
    auto zero_acc = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[j][e] = 0.f;
    };

    // staging: thread t owns float4 column t % 16 of patch rows 2u + rp of channel (t / 16) % 8, rp = t / 128
    // (WIDE 1: column t % 32 of patch row u of channel t / 32; WIDE 2: column t % 64 of patch row u / 2 of channel 4 (u % 2) + t / 64)
    const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
    const int pq = tid & (LPRK - 1), xc = WIDE == 2 ? wave : (tid / LPRK) & (CC - 1), rp = WIDE ? 0 : wave >> 1;  // rp, and with WIDE 2 xc, scalar: row tests and row pointers stay on the SALU
    // patch row and additional channels of staging pass u
    auto pass_row = [&](int u) __attribute__((always_inline)) { return WIDE == 2 ? u >> 1 : WIDE == 1 ? u : 2 * u + rp; };
    auto pass_ch = [&](int u) __attribute__((always_inline)) { return WIDE == 2 ? 4 * (u & 1) : 0; };
    const bool x_lane = pq < ((p.W + 3) >> 2);
    const int xcol = min(4 * pq, p.W - 4);
    const uint32_t x_off = x_lane ? (uint32_t)(xc * p.H * p.W + xcol) * 4u : 0u;
    const int x_dst0 = xc * PPLANE + p.pw + xcol;
    float4 Av[2][KK], xv[NXP];
    // loads of stage (tile geometry in b / iy_base / mb, chunk ch): the A values into register set SET, the patch rows into xv
    auto prefetch = [&](auto set_c, int ch) __attribute__((always_inline)) {
        constexpr int SET = decltype(set_c)::value;
        const float* asrc = p.wimg + ((i64)mb * p.nchunks + ch) * AIMG;
#pragma unroll
        for (int u = 0; u < KK; ++u) Av[SET][u] = ldg4(asrc + u * 256, (uint32_t)lane * 16u);
        const float* xsrc = p.x + ((i64)b * p.C + (i64)ch * CC) * p.H * p.W;
#pragma unroll
        for (int u = 0; u < NXP; ++u) {
            const int r = pass_row(u), iy = iy_base + r;
            if (r < p.PR && iy >= 0 && iy < p.H) xv[u] = ldg4(xsrc + ((i64)pass_ch(u) * p.H + iy) * p.W, x_off);  // scalar test
            else xv[u] = zero4;
        }
    };
    auto park = [&](int buf) __attribute__((always_inline)) {
        int xd = x_dst0 + buf * PBUF;
        FX_PIN_VGPR(xd);
        if (x_lane) {
#pragma unroll
            for (int u = 0; u < NXP; ++u) {
                const int r = pass_row(u);
                if (r < p.PR) {  // scalar test
                    const float4 v = xv[u];
                    float* d = smem + xd + pass_ch(u) * PPLANE + r * p.PW;
                    d[0] = v.x; d[1] = v.y; d[2] = v.z; d[3] = v.w;
                }
            }
        }
    };
    // One stage: 9 taps x 4 channel pairs, fully unrolled; two B register sets alternate so that the LDS reads of step i+1
    // are in flight while the MFMAs of step i run.  The A value of step (tap t, pair cp) is component cp of Av[SET][t].
    auto compute = [&](auto set_c) __attribute__((always_inline)) {
        constexpr int SET = decltype(set_c)::value;
        float b0[TN], b1[TN];
#pragma unroll
        for (int ky = 0; ky < 3; ++ky)
#pragma unroll
            for (int j = 0; j < TN; ++j) FX_PIN_VGPR(boff[ky][j]);
        auto rd = [&](float (&bv)[TN], int step) __attribute__((always_inline)) {
            const int t = step >> 2, cp = step & 3, ky = t / 3, kx = t % 3;
            const int imm = (SET * PBUF + 2 * cp * PPLANE + kx) * 4;
#pragma unroll
            for (int j = 0; j < TN; ++j) bv[j] = *(const float*)((const char*)smem + boff[ky][j] + imm);
            __builtin_amdgcn_sched_barrier(0);
        };
        auto mma = [&](const float (&bv)[TN], int step) __attribute__((always_inline)) {
            const float a = f4sel(Av[SET][step >> 2], step & 3);
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, bv[j], acc[j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        };
        rd(b0, 0);
#pragma unroll
        for (int step = 0; step < KK * 4; step += 2) {
            rd(b1, step + 1);
            mma(b0, step);
            if (step + 2 < KK * 4) rd(b0, step + 2);
            mma(b1, step + 1);
        }
    };
    // The stores of a tile: a scalar base per accumulator row (SALU) and one 32-bit lane offset per pixel block, so that
    // a store costs no vector ALU work; tiles that reach past the last output channel or pixel take the checked path.
    // The bias of the 16 output rows this lane stores, loaded at the start of a tile's last stage: in flight under that stage's
    // MFMAs instead of between them and the stores (where every wave of the block would wait for it at the same time).
    float bv[16];
    auto load_bias = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const int m = m0 + wm * 32 + igemm::Mfma<float>::row(e, lane);
            bv[e] = BIAS ? p.bias[m < p.M ? m : p.M - 1] : 0.f;
        }
    };
    auto store_tile = [&]() __attribute__((always_inline)) {
        typedef __attribute__((address_space(1))) char gchar;
        typedef __attribute__((address_space(1))) float gfloat;
        const int mw = m0 + wm * 32;  // scalar
        float* const out = p.y + ((i64)b * p.M + mw) * p.L;
        const int wpix0 = pix0 + wn * 32 * TN;
        auto rows = [&](auto checked_c) __attribute__((always_inline)) {
            constexpr bool CHECKED = decltype(checked_c)::value;
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int pi = wpix0 + j * 32 + l32;
                const uint32_t lo = (uint32_t)(4 * half * p.L + pi) * 4u;
                if (!CHECKED || pi < p.L) {
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const int ru = 8 * (e / 4) + e % 4;  // row(e, lane) = ru + 4 * half
                        if (!CHECKED || mw + ru + 4 * half < p.M) {
                            float v = acc[j][e];
                            if (BIAS) {
                                v = v + bv[e];
                                if (p.relu) v = v > 0.f ? v : 0.f;
                            }
                            float* rowp = out + (i64)ru * p.L;
                            FX_PIN_SGPR(rowp);  // keeps the row base apart from the lane offset: scalar base + 32-bit offset
                            *(gfloat*)((gchar*)rowp + lo) = v;
                        }
                    }
                }
            }
        };
        if (mw + 32 <= p.M && wpix0 + 32 * TN <= p.L) rows(std::false_type());
        else rows(std::true_type());
    };

    int ch = 0;
    geo(q);
    prefetch(std::integral_constant<int, 0>(), 0);
    set_boff();
    zero_acc();
    __syncthreads();  // the zero fill is complete before the first patch lands on it
    park(0);
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0) on every path into the loop (see the end of a stage)
    __syncthreads();
    // stage with register / LDS set SET; returns false after the block's last stage
    auto stage = [&](auto set_c) __attribute__((always_inline)) -> bool {
        constexpr int SET = decltype(set_c)::value;
        const bool last_ch = ch + 1 == p.nchunks;
        const int nq = last_ch ? q + qstep : q, nch = last_ch ? 0 : ch + 1;
        const bool more = nq < qend;
        // the finished tile's coordinates are needed by its stores after the next tile's have been formed for the loads
        const int cb = b, cm0 = m0, cpix0 = pix0;
        if (BIAS && last_ch) load_bias();
        if (more) {
            if (last_ch) geo(nq);
            prefetch(std::integral_constant<int, SET ^ 1>(), nch);
        }
        compute(set_c);
        // The MFMAs issued last are still running while the patch is parked and the tile stored: a wave's matrix
        // instructions complete in the background of its own later instructions.
        if (more) park(SET ^ 1);
        // Parking waited for the newest loads, so every load has landed; saying so here, BEFORE the stores, keeps the
        // compiler from guarding the next stage's first MFMAs with waits and leaves the stores to drain under them.
        __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0), other counters untouched
        if (last_ch) {
            const int nb = b, nm0 = m0, npix0 = pix0;
            b = cb; m0 = cm0; pix0 = cpix0;
            store_tile();
            b = nb; m0 = nm0; pix0 = npix0;
            if (more) {
                set_boff();
                zero_acc();
            }
        }
        __syncthreads();
        q = nq;
        ch = nch;
        return more;
    };
    while (true) {
        if (!stage(std::integral_constant<int, 0>())) break;
        if (!stage(std::integral_constant<int, 1>())) break;
    }
}

struct Plan {
    bool ok = false;
    int WM = 4, TN = 0, PR = 0, PW = 0, PLANE = 0, tpi = 0, mtiles = 0, nchunks = 0;
    bool tall = false;  // more than 8 patch rows: the NXP_TALL instantiation
    bool narrow = false;  // more than 20 patch rows of at most 32 floats: the NARROW instantiation
    int nimg = 0, RPI = 0;  // small maps: images per tile and patch rows per image (0: one image per tile)
    i64 cost = 0;           // modelled cost: rounds of co-resident blocks x MFMA work of a block
    size_t smem = 0;
    bool persist = false;  // a plan for conv_patch_persist_kernel (persist_plan); PW is then its padded row pitch
    int wide = 0;          // its instantiation for rows of 65 to 128 floats (1) or 129 to 256 (2)
    int bm() const { return 32 * WM; }
    int npix() const { return 32 * TN * (4 / WM); }
    i64 wimg() const { return (i64)bm() * WPITCH; }
};

// The plan for one tile shape (wm x tn); false when the shape does not fit this layer.
inline bool shape_plan(Plan& pl, int wm, int tn, int num_cus, i64 B, i64 C, i64 H, i64 W, i64 M, i64 OH, i64 OW, i64 sh, i64 sw, i64 ph,
                       i64 pw) {
    const i64 L = OH * OW, slots = 2 * (i64)std::max(1, num_cus);
    const i64 bm = 32 * wm, np = 32 * tn * (4 / wm), tiles = fx::ceil_div(L, np), mtiles = fx::ceil_div(M, bm);
    // output rows under a tile: tiles that start on a row boundary cover exactly np / OW rows
    const i64 rows = std::min<i64>(OH, np % OW == 0 ? np / OW : (np - 1) / OW + 2), PR = (rows - 1) * sh + 3;
    const bool tall_ok = wm <= 2 || tn <= 6;  // instantiated tall variants
    const bool narrow_ok = W <= 2 * LPR && wm >= 2 && tall_ok;  // 21 to 40 patch rows: rows of at most 32 floats, four per staging pass
    // at most half of the channel rows and half of the pixels of an image's tiles may be padding (measured at 7 x 7 maps,
    // 49 pixels under a 128-pixel tile: 0.084 ms against 0.061 ms for the implicit GEMM at [256,128,7,7] -> 128)
    if (PR > (narrow_ok ? 4 : 2) * NXP_TALL || (PR > 2 * NXP_SHORT && !tall_ok) || mtiles * bm > M * 2 || tiles * np > L * 2) return false;
    // strided layers, whose patch is four times the tile: at most a third of the pixels may be padding (16 x 16 maps at stride 2,
    // 64 pixels under a 128-pixel tile: 57 and 62 against 68 and 95 TFLOP/s for the implicit GEMM at 64 -> 128 and 128 -> 256)
    if ((sh > 1 || sw > 1) && tiles * np * 2 > L * 3) return false;
    pl = Plan();
    pl.WM = wm; pl.TN = tn; pl.PR = (int)PR; pl.tpi = (int)tiles;
    pl.cost = fx::ceil_div(B * tiles * mtiles, slots) * np * bm;
    pl.tall = pl.PR > 2 * NXP_SHORT;
    pl.narrow = pl.PR > 2 * NXP_TALL;
    pl.PW = (int)(W + 2 * pw);
    pl.PLANE = wgp::odd_pitch(pl.PR * pl.PW);
    pl.smem = ((size_t)pl.wimg() + (size_t)CC * pl.PLANE + SLACK) * sizeof(float);
    pl.mtiles = (int)mtiles;
    pl.nchunks = (int)(C / CC);
    if (pl.smem > LDS_BUDGET || B * pl.tpi > 0x7fffffff || pl.mtiles > 65535) return false;
    pl.ok = true;
    return true;
}

// Tile shapes of the persistent variant (wm x tn).
constexpr int N_PSHAPES = 5;
static const int PSHAPES[N_PSHAPES][2] = {{4, 5}, {4, 4}, {2, 5}, {2, 4}, {2, 3}};
// The plan of the persistent variant for one tile shape; false when the shape does not fit this layer.
inline bool persist_plan(Plan& pl, int wm, int tn, int num_cus, i64 B, i64 C, i64 H, i64 W, i64 M, i64 OH, i64 OW, i64 sh, i64 sw, i64 ph,
                         i64 pw) {
    const i64 L = OH * OW, slots = 2 * (i64)std::max(1, num_cus);
    const i64 bm = 32 * wm, np = 32 * tn * (4 / wm), tiles = fx::ceil_div(L, np), mtiles = fx::ceil_div(M, bm);
    const i64 rows = std::min<i64>(OH, np % OW == 0 ? np / OW : (np - 1) / OW + 2), PR = (rows - 1) * sh + 3;
    const int wide = W > 8 * LPR ? 2 : W > 4 * LPR ? 1 : 0;  // wide rows: fewer patch rows, and a register budget without the fifth accumulator block
    // wide rows have no 32-row tile: a 64-row tile over 32 channels measured 48 against 67 TFLOP/s for the implicit GEMM
    // ([16,64,112,112] <- 32 data gradient), so at most a third of the rows may be padding there
    if (wide && mtiles * bm * 2 > M * 3) return false;
    if (PR > (wide == 2 ? NXP_WIDE2 / 2 : wide ? NXP_WIDE : 2 * NXP_PERSIST) || (wide && tn > 4) || mtiles * bm > M * 2 || tiles * np > L * 2 || B * tiles * mtiles > 0x7fffffff)
        return false;
    // patch row pitch: with unit column stride a run of 32 pixels that wraps to the next output row must continue 32
    // words further on (sh * pitch - OW a multiple of 32), else two of its lanes share a bank; the plain pitch when that
    // does not fit the plane.
    i64 pw2 = W + 2 * pw;
    if (sw == 1) {
        i64 padded = pw2;
        while ((sh * padded - OW) % 32 != 0) ++padded;
        if (PR * padded <= PPLANE) pw2 = padded;
    }
    if (PR * pw2 > PPLANE) return false;
    pl = Plan();
    pl.persist = true;
    pl.wide = wide;
    pl.WM = wm; pl.TN = tn; pl.PR = (int)PR; pl.tpi = (int)tiles; pl.PW = (int)pw2; pl.PLANE = PPLANE;
    pl.mtiles = (int)mtiles;
    pl.nchunks = (int)(C / CC);
    pl.cost = fx::ceil_div(B * tiles * mtiles, slots) * np * bm;
    pl.smem = PP_LDS;
    pl.ok = true;
    return true;
}

// C input channels of H x W, M output channels of OH x OW (already the dimensions of the pass that runs).
// Among the tile shapes whose patch fits, takes the one with the least (rounds of co-resident blocks) x (work of
// a block): padded pixels, padded channels and a nearly empty last round all cost MFMA time.
inline Plan make_plan(int num_cus, i64 B, i64 C, i64 H, i64 W, i64 M, i64 OH, i64 OW, i64 kh, i64 kw, i64 sh, i64 sw, i64 ph,
                      i64 pw) {
    Plan pl;
    if (kh != 3 || kw != 3 || C % CC != 0 || W < 4 || W > 16 * LPR || sh > 8 || sw > 8) return pl;
    const i64 L = OH * OW;
    // Maps of at most 64 pixels: a 128-pixel tile takes as many whole images as fit its pixels and the 20 patch rows
    // (8 x 8 and 7 x 7 maps: two images), provided that fills at least half of the tile.
    const i64 RPI = (OH - 1) * sh + 3;
    if (L <= 64 && B >= 2 && W <= 4 * LPR) {  // (its staging covers rows of at most 64 floats)
        // up to 40 patch rows where the NARROW staging pays: strided layers, and rows of at least two vectors (5 x 5 and 6 x 6 maps
        // at stride 1, five and three images per tile: 79-100 and 71-97 TFLOP/s against 66-85 and 72-104 for the implicit GEMM over
        // 64 to 256 channels; 4 x 4 maps, one vector per row in eight lanes: 48-65 against 59-104, left to the implicit GEMM)
        const bool narrow_rows = W <= 2 * LPR && (sh > 1 || sw > 1 || W >= 5);
        const i64 nimg = std::min<i64>(std::min<i64>(128 / L, (narrow_rows ? 4 : 2) * NXP_TALL / RPI), B);
        const int wm = M > 64 ? 4 : 2;
        const i64 bm = 32 * wm, mtiles = fx::ceil_div(M, bm);
        if (nimg >= 2 && nimg * L >= 64 && mtiles * bm <= M * 2 && mtiles <= 65535) {
            pl.WM = wm; pl.TN = wm == 4 ? 4 : 2;
            pl.nimg = (int)nimg; pl.RPI = (int)RPI;
            pl.PR = (int)(nimg * RPI);
            pl.tall = true;
            pl.narrow = pl.PR > 2 * NXP_TALL;
            pl.tpi = 1;
            pl.PW = (int)(W + 2 * pw);
            pl.PLANE = wgp::odd_pitch(pl.PR * pl.PW);
            pl.smem = ((size_t)pl.wimg() + (size_t)CC * pl.PLANE + SLACK) * sizeof(float);
            pl.mtiles = (int)mtiles;
            pl.nchunks = (int)(C / CC);
            pl.ok = pl.smem <= LDS_BUDGET;
            return pl;
        }
    }
    static const int shapes[11][2] = {{4, 8}, {4, 7}, {4, 6}, {4, 5}, {4, 4}, {2, 4}, {2, 3}, {2, 2}, {1, 4}, {1, 3}, {1, 2}};
    Plan best;
    for (const auto& sp : PSHAPES) {
        Plan q;
        if (persist_plan(q, sp[0], sp[1], num_cus, B, C, H, W, M, OH, OW, sh, sw, ph, pw) && (!best.ok || q.cost < best.cost)) best = q;
    }
    for (const auto& sp : shapes) {
        Plan q;
        if (W <= 4 * LPR && shape_plan(q, sp[0], sp[1], num_cus, B, C, H, W, M, OH, OW, sh, sw, ph, pw) && (!best.ok || q.cost < best.cost)) best = q;
    }
    return best;
}

// Every tile shape whose modelled cost is within 1.5 x of the best one: the candidates that run() times once per layer
// shape (the model counts MFMA work and rounds of blocks; staging, weight-image size and LDS traffic per MFMA differ
// between shapes by more than that: measured spreads of 25 % and more between shapes of equal modelled cost).
constexpr int MAX_CAND = 11 + N_PSHAPES;
inline int candidates(Plan (&out)[MAX_CAND], int num_cus, i64 B, i64 C, i64 H, i64 W, i64 M, i64 OH, i64 OW, i64 sh, i64 sw, i64 ph, i64 pw) {
    static const int shapes[11][2] = {{4, 8}, {4, 7}, {4, 6}, {4, 5}, {4, 4}, {2, 4}, {2, 3}, {2, 2}, {1, 4}, {1, 3}, {1, 2}};
    Plan all[MAX_CAND];
    int n = 0;
    i64 best = -1;
    for (const auto& sp : PSHAPES)
        if (persist_plan(all[n], sp[0], sp[1], num_cus, B, C, H, W, M, OH, OW, sh, sw, ph, pw)) {
            if (best < 0 || all[n].cost < best) best = all[n].cost;
            ++n;
        }
    for (const auto& sp : shapes)
        if (W <= 4 * LPR && shape_plan(all[n], sp[0], sp[1], num_cus, B, C, H, W, M, OH, OW, sh, sw, ph, pw)) {
            if (best < 0 || all[n].cost < best) best = all[n].cost;
            ++n;
        }
    int m = 0;
    for (int k = 0; k < n; ++k)
        if (all[k].cost * 2 <= best * 3) out[m++] = all[k];
    return m;
}
inline int plan_code(const Plan& pl) { return pl.WM * 16 + pl.TN + (pl.persist ? 256 : 0); }

// Sized for 128-row images whatever tile was picked, so the figure does not depend on the CU count behind the plan.
inline i64 workspace_bytes(const Plan& pl, i64 M) { return fx::ceil_div(M, (i64)128) * 128 * WPITCH * pl.nchunks * (i64)sizeof(float); }

// w is the reference's [Cout][Cin][3][3] filter; flip selects the data-gradient image.
// The persistent variant for plan pl (pl.persist).
inline int launch_persist(fx_ctx* c, const Plan& pl, const float* x, const float* w, float* y, float* wimg, int flip, i64 Cout, i64 Cin,
                          i64 B, i64 C, i64 H, i64 W, i64 M, i64 OH, i64 OW, i64 sh, i64 sw, i64 ph, i64 pw, const float* bias, int relu) {
    const i64 mblocks = (i64)pl.mtiles * pl.WM;
    const i64 n = mblocks * pl.nchunks * KK * 64 * 4;
    FX_LAUNCH(dim3((unsigned)fx::ceil_div(n, 256)), dim3(256), 0, c->stream, (w, wimg, (int)Cout, (int)Cin, (int)M, pl.nchunks, flip, n), wimg2_kernel);
    FX_LAUNCH_CHECK();
    Params p;
    p.x = x; p.wimg = wimg; p.y = y; p.bias = bias; p.relu = relu;
    p.C = (int)C; p.H = (int)H; p.W = (int)W; p.M = (int)M; p.OH = (int)OH; p.OW = (int)OW;
    p.sh = (int)sh; p.sw = (int)sw; p.ph = (int)ph; p.pw = (int)pw;
    p.PR = pl.PR; p.PW = pl.PW; p.PLANE = PPLANE; p.L = (int)(OH * OW); p.tpi = pl.tpi; p.nchunks = pl.nchunks;
    p.div_tpi = FastDiv((uint32_t)pl.tpi);
    p.div_ow = FastDiv((uint32_t)OW);
    p.nimg = 0; p.RPI = 0; p.B = (int)B;
    p.bt = (int)(B * pl.tpi);
    p.ntiles = (int)(B * pl.tpi * pl.mtiles);
    p.bufsz = PBUF;
    p.div_bt = FastDiv((uint32_t)p.bt);
    int nblk = std::min(p.ntiles, 2 * std::max(1, c->num_cus));  // two blocks per CU
    p.xcd_chunk = 0;
    if (p.ntiles % 8 == 0 && nblk >= 8) {
        nblk -= nblk % 8;
        p.xcd_chunk = p.ntiles / 8;
    }
    const dim3 grid((unsigned)nblk);
#define FX_CPK_PERSIST(WMV, TNV, WIDEV)                                                                                    \
    case WIDEV * 256 + WMV * 16 + TNV: {                                                                                \
        static const hipError_t attr0 = hipFuncSetAttribute((const void*)conv_patch_persist_kernel<WMV, TNV, false, WIDEV>,   \
                                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)PP_LDS);         \
        static const hipError_t attr1 = hipFuncSetAttribute((const void*)conv_patch_persist_kernel<WMV, TNV, true, WIDEV>,    \
                                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)PP_LDS);         \
        FX_HIP_CHECK(attr0);                                                                                                  \
        FX_HIP_CHECK(attr1);                                                                                                  \
        if (bias) FX_LAUNCH(grid, dim3(NT), PP_LDS, c->stream, (p), conv_patch_persist_kernel<WMV, TNV, true, WIDEV>);        \
        else FX_LAUNCH(grid, dim3(NT), PP_LDS, c->stream, (p), conv_patch_persist_kernel<WMV, TNV, false, WIDEV>);            \
    } break;
    switch (pl.wide * 256 + pl.WM * 16 + pl.TN) {
        FX_CPK_PERSIST(4, 5, 0)
        FX_CPK_PERSIST(4, 4, 0)
        FX_CPK_PERSIST(2, 5, 0)
        FX_CPK_PERSIST(2, 4, 0)
        FX_CPK_PERSIST(2, 3, 0)
        FX_CPK_PERSIST(4, 4, 1)
        FX_CPK_PERSIST(2, 4, 1)
        FX_CPK_PERSIST(2, 3, 1)
        FX_CPK_PERSIST(4, 4, 2)
        FX_CPK_PERSIST(2, 4, 2)
        FX_CPK_PERSIST(2, 3, 2)
        default: FX_REQUIRE(false, "conv patch kernel (persistent): unexpected tile %d x %d", pl.WM, pl.TN);
    }
#undef FX_CPK_PERSIST
    FX_LAUNCH_CHECK();
    return FX_OK;
}

inline int launch_plan(fx_ctx* c, const Plan& pl, const float* x, const float* w, float* y, float* wimg, int flip, i64 Cout, i64 Cin, i64 B,
                       i64 C, i64 H, i64 W, i64 M, i64 OH, i64 OW, i64 sh, i64 sw, i64 ph, i64 pw, const float* bias, int relu) {
    if (pl.persist) return launch_persist(c, pl, x, w, y, wimg, flip, Cout, Cin, B, C, H, W, M, OH, OW, sh, sw, ph, pw, bias, relu);
    const i64 n = (i64)pl.mtiles * pl.nchunks * pl.wimg();
    FX_LAUNCH(dim3((unsigned)fx::ceil_div(n, 256)), dim3(256), 0, c->stream, (w, wimg, (int)Cout, (int)Cin, (int)M, pl.bm(),
                                                                                  pl.nchunks, flip, n), wimg_kernel);
    FX_LAUNCH_CHECK();
    Params p;
    p.x = x; p.wimg = wimg; p.y = y; p.bias = bias; p.relu = relu;
    p.C = (int)C; p.H = (int)H; p.W = (int)W; p.M = (int)M; p.OH = (int)OH; p.OW = (int)OW;
    p.sh = (int)sh; p.sw = (int)sw; p.ph = (int)ph; p.pw = (int)pw;
    p.PR = pl.PR; p.PW = pl.PW; p.PLANE = pl.PLANE; p.L = (int)(OH * OW); p.tpi = pl.tpi; p.nchunks = pl.nchunks;
    p.div_tpi = FastDiv((uint32_t)pl.tpi);
    p.div_ow = FastDiv((uint32_t)OW);
    p.nimg = pl.nimg; p.RPI = pl.RPI; p.B = (int)B;
    p.div_L = FastDiv((uint32_t)(OH * OW));
    p.div_rpi = FastDiv((uint32_t)std::max(1, pl.RPI));
    const i64 gx = pl.nimg ? fx::ceil_div(B, (i64)pl.nimg) : B * pl.tpi;
    const dim3 grid((unsigned)gx, (unsigned)pl.mtiles);
    p.xcd_chunk = gx % 8 == 0 ? (int)(gx / 8) : 0;
    if (pl.nimg) {
#define FX_CPK_LAUNCH_MULTI(WMV, TNV, NARROWV)                                                                       \
    {                                                                                                                 \
        static const hipError_t attr0 = hipFuncSetAttribute((const void*)conv_patch_kernel<WMV, TNV, false, NXP_TALL, true, NARROWV>, \
                                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_BUDGET); \
        static const hipError_t attr1 = hipFuncSetAttribute((const void*)conv_patch_kernel<WMV, TNV, true, NXP_TALL, true, NARROWV>, \
                                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_BUDGET); \
        FX_HIP_CHECK(attr0);                                                                                          \
        FX_HIP_CHECK(attr1);                                                                                          \
        if (bias) FX_LAUNCH(grid, dim3(NT), pl.smem, c->stream, (p), conv_patch_kernel<WMV, TNV, true, NXP_TALL, true, NARROWV>);  \
        else FX_LAUNCH(grid, dim3(NT), pl.smem, c->stream, (p), conv_patch_kernel<WMV, TNV, false, NXP_TALL, true, NARROWV>);      \
    }
        if (pl.narrow) {
            if (pl.WM == 4) FX_CPK_LAUNCH_MULTI(4, 4, true) else FX_CPK_LAUNCH_MULTI(2, 2, true)
        } else {
            if (pl.WM == 4) FX_CPK_LAUNCH_MULTI(4, 4, false) else FX_CPK_LAUNCH_MULTI(2, 2, false)
        }
#undef FX_CPK_LAUNCH_MULTI
        FX_LAUNCH_CHECK();
        return FX_OK;
    }
#define FX_CPK_LAUNCH_N(WMV, TNV, NXPV, NARROWV)                                                                     \
    {                                                                                                                 \
        static const hipError_t attr0 = hipFuncSetAttribute((const void*)conv_patch_kernel<WMV, TNV, false, NXPV, false, NARROWV>, \
                                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_BUDGET); \
        static const hipError_t attr1 = hipFuncSetAttribute((const void*)conv_patch_kernel<WMV, TNV, true, NXPV, false, NARROWV>, \
                                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_BUDGET); \
        FX_HIP_CHECK(attr0);                                                                                          \
        FX_HIP_CHECK(attr1);                                                                                          \
        if (bias) FX_LAUNCH(grid, dim3(NT), pl.smem, c->stream, (p), conv_patch_kernel<WMV, TNV, true, NXPV, false, NARROWV>);  \
        else FX_LAUNCH(grid, dim3(NT), pl.smem, c->stream, (p), conv_patch_kernel<WMV, TNV, false, NXPV, false, NARROWV>);      \
    }
#define FX_CPK_LAUNCH(WMV, TNV)                                                                                       \
    case WMV * 16 + TNV:                                                                                              \
        if (pl.narrow) FX_CPK_LAUNCH_N(WMV, TNV, NXP_TALL, true)                                                      \
        else if (pl.tall) FX_CPK_LAUNCH_N(WMV, TNV, NXP_TALL, false)                                                  \
        else FX_CPK_LAUNCH_N(WMV, TNV, NXP_SHORT, false)                                                              \
        break;
#define FX_CPK_LAUNCH_WIDE_TILE(WMV, TNV) /* one block of channels: no NARROW instantiation */                       \
    case WMV * 16 + TNV:                                                                                              \
        FX_REQUIRE(!pl.narrow, "conv patch kernel: no narrow-row variant of tile %d x %d", WMV, TNV);                \
        if (pl.tall) FX_CPK_LAUNCH_N(WMV, TNV, NXP_TALL, false) else FX_CPK_LAUNCH_N(WMV, TNV, NXP_SHORT, false)      \
        break;
#define FX_CPK_LAUNCH_SHORT(WMV, TNV)                                                                                 \
    case WMV * 16 + TNV:                                                                                              \
        FX_REQUIRE(!pl.tall, "conv patch kernel: no tall variant of tile %d x %d", WMV, TNV);                        \
        FX_CPK_LAUNCH_N(WMV, TNV, NXP_SHORT, false)                                                                   \
        break;
    switch (pl.WM * 16 + pl.TN) {
        FX_CPK_LAUNCH(4, 4)
        FX_CPK_LAUNCH(4, 5)
        FX_CPK_LAUNCH(4, 6)
        FX_CPK_LAUNCH_SHORT(4, 7)
        FX_CPK_LAUNCH_SHORT(4, 8)
        FX_CPK_LAUNCH(2, 2)
        FX_CPK_LAUNCH(2, 3)
        FX_CPK_LAUNCH(2, 4)
        FX_CPK_LAUNCH_WIDE_TILE(1, 2)
        FX_CPK_LAUNCH_WIDE_TILE(1, 3)
        FX_CPK_LAUNCH_WIDE_TILE(1, 4)
        default: FX_REQUIRE(false, "conv patch kernel: unexpected tile %d x %d", pl.WM, pl.TN);
    }
#undef FX_CPK_LAUNCH_N
#undef FX_CPK_LAUNCH_WIDE_TILE
#undef FX_CPK_LAUNCH_SHORT
#undef FX_CPK_LAUNCH
    FX_LAUNCH_CHECK();
    return FX_OK;
}

// Runs the layer with the tile shape that measured fastest for this layer shape on this device.  The first call for a
// layer (filter, map and channel sizes, stride, padding, epilogue) and batch size class (floor(log2(B)): a ragged last batch
// shares the class of its neighbours or costs one more timing, never one per distinct size) times the candidate shapes (each
// writes the same, complete output: the order of every output's sum does not depend on the tile shape) and remembers the
// winner in the context; fx_conv2d_tune times again whatever the cache holds.  Nothing is timed when the output overlaps an operand (the repeated launches would read
// what an earlier one wrote), and FX_CONV_TUNE=0 keeps the modelled choice everywhere.
inline int batch_class(i64 B) {
    int k = 0;
    while ((i64(2) << k) <= B) ++k;
    return k;
}
inline bool ranges_overlap(const void* a, i64 a_bytes, const void* b, i64 b_bytes) {
    const uintptr_t a0 = (uintptr_t)a, b0 = (uintptr_t)b;
    return a0 < b0 + (uintptr_t)b_bytes && b0 < a0 + (uintptr_t)a_bytes;
}
inline int run(fx_ctx* c, const Plan& pl, const float* x, const float* w, float* y, float* wimg, int flip, i64 Cout, i64 Cin, i64 B,
               i64 C, i64 H, i64 W, i64 M, i64 OH, i64 OW, i64 sh, i64 sw, i64 ph, i64 pw, const float* bias = nullptr, int relu = 0) {
    static const bool tune = [] { const char* v = getenv("FX_CONV_TUNE"); return !(v && atoi(v) == 0); }();
    if (!tune || pl.nimg) return launch_plan(c, pl, x, w, y, wimg, flip, Cout, Cin, B, C, H, W, M, OH, OW, sh, sw, ph, pw, bias, relu);
    const std::array<i64, 14> key = {flip, batch_class(B), C, H, W, M, OH, OW, sh, sw, ph, pw, bias ? 1 : 0, relu};
    // a stream that is recording a graph cannot be timed: a layer shape first met there runs with the modelled tile
    if (c->capturing && c->conv_tile_cache.find(key) == c->conv_tile_cache.end())
        return launch_plan(c, pl, x, w, y, wimg, flip, Cout, Cin, B, C, H, W, M, OH, OW, sh, sw, ph, pw, bias, relu);
    Plan cand[MAX_CAND];
    const int n = candidates(cand, c->num_cus, B, C, H, W, M, OH, OW, sh, sw, ph, pw);
    auto it = c->conv_tile_cache.find(key);
    if (c->conv_tile_cache.size() > 4096) {  // layer shapes of a process are few; a runaway caller does not grow the table for ever
        c->conv_tile_cache.clear();
        it = c->conv_tile_cache.end();
    }
    if (it != c->conv_tile_cache.end() && c->conv_retune) {
        c->conv_tile_cache.erase(it);
        it = c->conv_tile_cache.end();
    }
    if (it == c->conv_tile_cache.end()) {
        const i64 y_bytes = B * M * OH * OW * 4;
        if (ranges_overlap(y, y_bytes, x, B * C * H * W * 4) || ranges_overlap(y, y_bytes, w, Cout * Cin * 9 * 4) ||
            (bias && ranges_overlap(y, y_bytes, bias, M * 4)))
            return launch_plan(c, pl, x, w, y, wimg, flip, Cout, Cin, B, C, H, W, M, OH, OW, sh, sw, ph, pw, bias, relu);
        int best = -1, n_last = n - 1;  // n_last: the candidate launched last
        if (n > 1) {
            if (!c->ev_tune[0]) {
                FX_HIP_CHECK(hipEventCreate(&c->ev_tune[0]));
                FX_HIP_CHECK(hipEventCreate(&c->ev_tune[1]));
            }
            // the modelled choice stays unless another shape is at least 5 % faster (timer noise between equals)
            int model = 0;
            for (int k = 1; k < n; ++k)
                if (cand[k].cost < cand[model].cost) model = k;
            float ms_of[MAX_CAND];
            auto time_one = [&](int k, float* ms) -> int {  // one warm-up launch, then three timed ones
                if (int rc = launch_plan(c, cand[k], x, w, y, wimg, flip, Cout, Cin, B, C, H, W, M, OH, OW, sh, sw, ph, pw, bias, relu)) return rc;
                FX_HIP_CHECK(hipEventRecord(c->ev_tune[0], c->stream));
                for (int rep = 0; rep < 3; ++rep)
                    if (int rc = launch_plan(c, cand[k], x, w, y, wimg, flip, Cout, Cin, B, C, H, W, M, OH, OW, sh, sw, ph, pw, bias, relu)) return rc;
                FX_HIP_CHECK(hipEventRecord(c->ev_tune[1], c->stream));
                FX_HIP_CHECK(hipEventSynchronize(c->ev_tune[1]));
                FX_HIP_CHECK(hipEventElapsedTime(ms, c->ev_tune[0], c->ev_tune[1]));
                return FX_OK;
            };
            for (int k = 0; k < n; ++k)
                if (int rc = time_one(k, &ms_of[k])) return rc;
            best = model;
            for (int k = 0; k < n; ++k)
                if (ms_of[k] < 0.95f * ms_of[best]) best = k;
            static const bool verbose = [] { const char* v = getenv("FX_CONV_VERBOSE"); return v && atoi(v) != 0; }();
            if (verbose)
                for (int k = 0; k < n; ++k)
                    fprintf(stderr, "[ferrox_hip] conv3x3 %s C=%lld %lldx%lld M=%lld: tile %dx%d%s %.4f ms%s%s\n", flip ? "dgrad" : "fwd", (long long)C,
                            (long long)H, (long long)W, (long long)M, cand[k].WM, cand[k].TN, cand[k].persist ? " persistent" : "", ms_of[k] / 3,
                            k == model ? " (model)" : "", k == best ? " (fastest)" : "");
            if (best != model) {  // a challenger has to win a second time against the modelled shape
                float again_model = 0.f, again_best = 0.f;
                if (int rc = time_one(model, &again_model)) return rc;
                if (int rc = time_one(best, &again_best)) return rc;
                n_last = best;  // the challenger was launched last
                if (!(again_best < 0.95f * again_model)) best = model;
            }
        }
        const int code = plan_code(best >= 0 ? cand[best] : pl);
        it = c->conv_tile_cache.emplace(key, code).first;
        if (best >= 0 && best == n_last) return FX_OK;  // the candidate launched last is the winner: its output stands
    }
    for (int k = 0; k < n; ++k)
        if (plan_code(cand[k]) == it->second)
            return launch_plan(c, cand[k], x, w, y, wimg, flip, Cout, Cin, B, C, H, W, M, OH, OW, sh, sw, ph, pw, bias, relu);
    return launch_plan(c, pl, x, w, y, wimg, flip, Cout, Cin, B, C, H, W, M, OH, OW, sh, sw, ph, pw, bias, relu);
}

}  // namespace cpk
