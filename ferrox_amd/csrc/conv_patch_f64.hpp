// 3x3 convolution forward (f64) on v_mfma_f64_16x16x4_f64 with the input patch staged in LDS and the weights held in
// registers; the stride-1 data gradient runs through the same kernel as a forward pass over grad_out with flipped,
// transposed weights.  The f64 twin of cpk::conv_patch_persist_kernel (conv_patch.hpp), same product
//   y[b][m][oy][ox] = sum over (c, ky, kx) of wgt[m][c][ky][kx] * in[b][c][oy*sh+ky-ph][ox*sw+kx-pw]
// (filter_2d . im2col(x) in the reference, src/backend/storage/extensions/convolutions.rs:218-290).
//
// The f64 MFMA multiplies a 16 x 4 by a 4 x 16 block in 64 cycles: lane l holds A[m = l%16][k = l/16] and
// B[k = l/16][n = l%16], one double each, and 4 of the 16 x 16 results (row 4e + l/16, column l%16).
// A block is 4 waves = 64 output channels (16 per wave) x 16 TN consecutive output pixels of one image, shared by the four
// waves; it walks the input channels in chunks of 8 (one stage each).  A stage is 9 taps x 2 groups of 4 channels = 18
// k-steps of TN MFMAs per wave.  Per stage
//   * a lane fetches the 18 A values of its output-channel row as nine 16-byte global loads (both channel groups of a tap
//     sit side by side in an image built once per call by wimg_kernel), one stage ahead, into one of two register sets;
//   * the block parks the zero-padded input rows under its pixel tile, 8 channel planes, in one of two LDS buffers; every
//     tap reads that patch at a shifted address: ds_read_b64 with the buffer, channel group and filter column in the
//     offset field, one read per MFMA.
// Blocks are persistent (two per CU) and keep the stage pipeline running across tile boundaries.
#pragma once
#include <cstdlib>

#include "igemm_core.hpp"

namespace cpd {
using igemm::FastDiv;
using igemm::f64x4;

constexpr int CC = 8, NT = 256, KK = 9;
constexpr int NXP = 8;     // patch rows: one per staging pass (32 lanes x 16 bytes cover a row of up to 64 doubles)
constexpr int LPR = 32;    // lanes per patch row
constexpr int SLACK = 16;
// plane pitch and buffer size in doubles, compile-time constants so that they ride in the 16-bit offset field of a read:
// 2 x (8 x 573 + 16) x 8 bytes = 73600 <= 72 KB per block (two blocks per CU)
constexpr int PPLANE = 573, PBUF = CC * PPLANE + SLACK;
constexpr size_t LDS_BYTES = 2 * (size_t)PBUF * sizeof(double);
static_assert(LDS_BYTES <= 72 * 1024 && (PBUF + 4 * PPLANE + 2) * 8 < 65536, "patch buffers");
constexpr int AIMG = KK * 64 * 2;  // doubles of one (16-row block, chunk) weight image

struct Params {
    const double* x;
    const double* wimg;
    double* y;
    const double* bias;  // optional, per output channel; with relu != 0 the sum is clamped at 0 afterwards
    int relu;
    int C, H, W, M, OH, OW, sh, sw, ph, pw;
    int PR, PW, L, tpi, nchunks;
    int xcd_chunk;  // tiles / 8 when that divides: workgroup ids go to the 8 XCDs round-robin, see the kernel
    int ntiles, bt;
    FastDiv div_tpi, div_ow, div_bt;
};

// Weight images in MFMA operand order: out[mb][ch][tap][lane][cp] = wgt[m = 16 mb + lane%16][c = 8 ch + 4 cp + lane/16][tap],
// zero in rows past M.  flip == 0 (forward): wgt[m][c][tap] = w[oc = m][c][tap]; flip == 1 (data gradient):
// wgt[m][c][tap] = w[oc = c][cin = m][8 - tap].
__global__ __launch_bounds__(256) void wimg_kernel(const double* __restrict__ w, double* __restrict__ out, int Cout, int Cin, int M,
                                                   int nchunks, int flip, i64 n) {
    const i64 i = (i64)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const int cp = (int)(i & 1), lane = (int)((i >> 1) & 63);
    i64 r = i >> 7;
    const int t = (int)(r % KK);
    r /= KK;
    const int ch = (int)(r % nchunks), mb = (int)(r / nchunks);
    const int mm = mb * 16 + (lane & 15), c = ch * CC + 4 * cp + (lane >> 4);
    double v = 0.;
    if (mm < M) v = flip ? w[((i64)c * Cin + mm) * KK + (KK - 1 - t)] : w[((i64)mm * Cin + c) * KK + t];
    out[i] = v;
}

__device__ __forceinline__ double2 ldg2(const double* base, uint32_t byteoff) {
    typedef __attribute__((address_space(1))) const char gchar;
    typedef double v2 __attribute__((ext_vector_type(2)));
    typedef __attribute__((address_space(1))) const v2 gv2;
    const v2 v = *(gv2*)((gchar*)base + byteoff);
    return make_double2(v.x, v.y);
}

template <int TN, bool BIAS>
__global__ __launch_bounds__(NT, 2) void conv_patch_f64_kernel(const Params p) {
    constexpr int BM = 64, NPIX = 16 * TN;
    FX_DYNAMIC_SMEM(double, smem);
    const int tid = threadIdx.x, lane = tid & 63, kq = lane >> 4, l16 = lane & 15;
    // in a scalar register: what derives from the wave index (rows, pointers, tests) stays on the scalar unit
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // this block's tiles: XCD x (workgroup ids go to the 8 XCDs round-robin) owns the contiguous range [x*chunk, (x+1)*chunk)
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
    for (int i = tid; i < 2 * PBUF; i += NT) smem[i] = 0.;  // the padding columns of both buffers stay zero from here on

    int b, m0, pix0, iy_base, py0, mb;
    auto geo = [&](int qq) __attribute__((always_inline)) {
        const int mt = (int)p.div_bt.div((uint32_t)qq), rem = qq - mt * p.bt;
        b = (int)p.div_tpi.div((uint32_t)rem);
        pix0 = (rem - b * p.tpi) * NPIX;
        py0 = (int)p.div_ow.div((uint32_t)pix0);
        iy_base = py0 * p.sh - p.ph;
        m0 = mt * BM;
        mb = mt * 4 + wave;
    };
    // byte offsets into a patch buffer of this lane's B operands, one set per filter row
    int boff[3][TN];
    auto set_boff = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int pi = pix0 + j * 16 + l16;
            const int py = (int)p.div_ow.div((uint32_t)pi), px = pi - py * p.OW;
            const int o = (pi < p.L ? (py - py0) * p.sh * p.PW + px * p.sw : 0) + kq * PPLANE;
#pragma unroll
            for (int ky = 0; ky < 3; ++ky) boff[ky][j] = (o + ky * p.PW) * 8;
        }
    };
    f64x4 acc[TN];
    auto zero_acc = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[j][e] = 0.;
    };

    // staging: thread t owns the pair of doubles t % 32 of patch row u of channel t / 32, u = 0 .. PR-1
    const double2 zero2 = make_double2(0., 0.);
    const int pq = tid & (LPR - 1), xc = wave * 2 + (lane >> 5);
    const bool x_lane = pq < ((p.W + 1) >> 1);
    const int xcol = min(2 * pq, p.W - 2);
    const uint32_t x_off = x_lane ? (uint32_t)(xc * p.H * p.W + xcol) * 8u : 0u;
    const int x_dst0 = xc * PPLANE + p.pw + xcol;
    double2 Av[2][KK], xv[NXP];
    auto prefetch = [&](auto set_c, int ch) __attribute__((always_inline)) {
        constexpr int SET = decltype(set_c)::value;
        const double* asrc = p.wimg + ((i64)mb * p.nchunks + ch) * AIMG;
#pragma unroll
        for (int u = 0; u < KK; ++u) Av[SET][u] = ldg2(asrc + u * 128, (uint32_t)lane * 16u);
        const double* xsrc = p.x + ((i64)b * p.C + (i64)ch * CC) * p.H * p.W;
#pragma unroll
        for (int u = 0; u < NXP; ++u) {
            const int iy = iy_base + u;
            if (u < p.PR && iy >= 0 && iy < p.H) xv[u] = ldg2(xsrc + (i64)iy * p.W, x_off);  // scalar test
            else xv[u] = zero2;
        }
    };
    auto park = [&](int buf) __attribute__((always_inline)) {
        int xd = x_dst0 + buf * PBUF;
        FX_PIN_VGPR(xd);
        if (x_lane) {
#pragma unroll
            for (int u = 0; u < NXP; ++u) {
                if (u < p.PR) {  // scalar test
                    double* d = smem + xd + u * p.PW;
                    d[0] = xv[u].x;
                    d[1] = xv[u].y;
                }
            }
        }
    };
    // One stage: 9 taps x 2 channel groups, fully unrolled; two B register sets alternate so that the LDS reads of step
    // i+1 are in flight while the MFMAs of step i run.  The A value of step (tap t, group cp) is component cp of Av[SET][t].
    auto compute = [&](auto set_c) __attribute__((always_inline)) {
        constexpr int SET = decltype(set_c)::value;
        double b0[TN], b1[TN];
#pragma unroll
        for (int ky = 0; ky < 3; ++ky)
#pragma unroll
            for (int j = 0; j < TN; ++j) FX_PIN_VGPR(boff[ky][j]);
        auto rd = [&](double (&bv)[TN], int step) __attribute__((always_inline)) {
            const int t = step >> 1, cp = step & 1, ky = t / 3, kx = t % 3;
            const int imm = (SET * PBUF + 4 * cp * PPLANE + kx) * 8;
#pragma unroll
            for (int j = 0; j < TN; ++j) bv[j] = *(const double*)((const char*)smem + boff[ky][j] + imm);
            __builtin_amdgcn_sched_barrier(0);
        };
        auto mma = [&](const double (&bv)[TN], int step) __attribute__((always_inline)) {
            const double a = (step & 1) ? Av[SET][step >> 1].y : Av[SET][step >> 1].x;
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[j] = __builtin_amdgcn_mfma_f64_16x16x4f64(a, bv[j], acc[j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        };
        rd(b0, 0);
#pragma unroll
        for (int step = 0; step < KK * 2; step += 2) {
            rd(b1, step + 1);
            mma(b0, step);
            if (step + 2 < KK * 2) rd(b0, step + 2);
            mma(b1, step + 1);
        }
    };
    // The stores of a tile: a scalar base per accumulator row group (SALU) and one 32-bit lane offset per pixel block.
    // The bias of the 4 output rows this lane stores, loaded at the start of a tile's last stage: in flight under that stage's
    // MFMAs instead of between them and the stores (where every wave of the block would wait for it at the same time).
    double bv[4];
    auto load_bias = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int m = m0 + wave * 16 + 4 * e + kq;
            bv[e] = BIAS ? p.bias[m < p.M ? m : p.M - 1] : 0.;
        }
    };
    auto store_tile = [&]() __attribute__((always_inline)) {
        typedef __attribute__((address_space(1))) char gchar;
        typedef __attribute__((address_space(1))) double gdouble;
        const int mw = m0 + wave * 16;  // scalar
        double* const out = p.y + ((i64)b * p.M + mw) * p.L;
        if (BIAS && TN >= 8) load_bias();
        auto rows = [&](auto checked_c) __attribute__((always_inline)) {
            constexpr bool CHECKED = decltype(checked_c)::value;
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int pi = pix0 + j * 16 + l16;
                const uint32_t lo = (uint32_t)(kq * p.L + pi) * 8u;
                if (!CHECKED || pi < p.L) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {  // row 4e + kq
                        if (!CHECKED || mw + 4 * e + kq < p.M) {
                            double v = acc[j][e];
                            if (BIAS) {
                                v = v + bv[e];
                                if (p.relu) v = v > 0. ? v : 0.;
                            }
                            double* rowp = out + (i64)(4 * e) * p.L;
                            FX_PIN_SGPR(rowp);  // keeps the row base apart from the lane offset: scalar base + 32-bit offset
                            *(gdouble*)((gchar*)rowp + lo) = v;
                        }
                    }
                }
            }
        };
        if (mw + 16 <= p.M && pix0 + NPIX <= p.L) rows(std::false_type());
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
    auto stage = [&](auto set_c) __attribute__((always_inline)) -> bool {
        constexpr int SET = decltype(set_c)::value;
        const bool last_ch = ch + 1 == p.nchunks;
        const int nq = last_ch ? q + qstep : q, nch = last_ch ? 0 : ch + 1;
        const bool more = nq < qend;
        // the finished tile's coordinates are needed by its stores after the next tile's have been formed for the loads
        const int cb = b, cm0 = m0, cpix0 = pix0;
        if (BIAS && last_ch && TN < 8) load_bias();  // the widest tile has no registers to spare during the stage
        if (more) {
            if (last_ch) geo(nq);
            prefetch(std::integral_constant<int, SET ^ 1>(), nch);
        }
        compute(set_c);
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
    int TN = 0, PR = 0, PW = 0, tpi = 0, mtiles = 0, nchunks = 0;
    i64 cost = 0;  // modelled cost: rounds of co-resident blocks x MFMA work of a block
};

constexpr int N_SHAPES = 3;
static const int SHAPES[N_SHAPES] = {8, 7, 5};

inline bool shape_plan(Plan& pl, int tn, int num_cus, i64 B, i64 C, i64 H, i64 W, i64 M, i64 OH, i64 OW, i64 sh, i64 sw, i64 ph, i64 pw) {
    const i64 L = OH * OW, slots = 2 * (i64)std::max(1, num_cus);
    const i64 np = 16 * tn, tiles = fx::ceil_div(L, np), mtiles = fx::ceil_div(M, (i64)64);
    const i64 rows = std::min<i64>(OH, np % OW == 0 ? np / OW : (np - 1) / OW + 2), PR = (rows - 1) * sh + 3;
    if (PR > NXP || mtiles * 64 > M * 2 || tiles * np > L * 2 || B * tiles * mtiles > 0x7fffffff) return false;
    // patch row pitch: with unit column stride a run of 16 pixels (16 doubles = all 32 banks) that wraps to the next output row
    // must continue 16 doubles further on (sh * pitch - OW a multiple of 16); the plain pitch when that does not fit
    i64 pw2 = W + 2 * pw;
    if (sw == 1) {
        i64 padded = pw2;
        while ((sh * padded - OW) % 16 != 0) ++padded;
        if (PR * padded <= PPLANE) pw2 = padded;
    }
    if (PR * pw2 > PPLANE) return false;
    pl = Plan();
    pl.ok = true;
    pl.TN = tn; pl.PR = (int)PR; pl.PW = (int)pw2; pl.tpi = (int)tiles; pl.mtiles = (int)mtiles; pl.nchunks = (int)(C / CC);
    pl.cost = fx::ceil_div(B * tiles * mtiles, slots) * np * 64;
    return true;
}

// C input channels of H x W, M output channels of OH x OW (already the dimensions of the pass that runs).
inline Plan make_plan(int num_cus, i64 B, i64 C, i64 H, i64 W, i64 M, i64 OH, i64 OW, i64 kh, i64 kw, i64 sh, i64 sw, i64 ph, i64 pw) {
    Plan best;
    if (kh != 3 || kw != 3 || C % CC != 0 || W < 2 || W % 2 != 0 || W > 2 * LPR || sh > 8 || sw > 8 || OH * OW < 64 || M < 32) return best;
    for (int tn : SHAPES) {
        Plan q;
        if (shape_plan(q, tn, num_cus, B, C, H, W, M, OH, OW, sh, sw, ph, pw) && (!best.ok || q.cost < best.cost)) best = q;
    }
    return best;
}

inline i64 workspace_bytes(const Plan& pl) { return (i64)pl.mtiles * 4 * pl.nchunks * AIMG * (i64)sizeof(double); }

// w is the reference's [Cout][Cin][3][3] filter; flip selects the data-gradient image.  x, wimg and y must be 16-byte aligned.
inline int run(fx_ctx* c, const Plan& pl, const double* x, const double* w, double* y, double* wimg, int flip, i64 Cout, i64 Cin, i64 B, i64 C,
               i64 H, i64 W, i64 M, i64 OH, i64 OW, i64 sh, i64 sw, i64 ph, i64 pw, const double* bias = nullptr, int relu = 0) {
    const i64 n = (i64)pl.mtiles * 4 * pl.nchunks * AIMG;
    FX_LAUNCH(dim3((unsigned)fx::ceil_div(n, 256)), dim3(256), 0, c->stream, (w, wimg, (int)Cout, (int)Cin, (int)M, pl.nchunks, flip, n), wimg_kernel);
    FX_LAUNCH_CHECK();
    Params p;
    p.x = x; p.wimg = wimg; p.y = y; p.bias = bias; p.relu = relu;
    p.C = (int)C; p.H = (int)H; p.W = (int)W; p.M = (int)M; p.OH = (int)OH; p.OW = (int)OW;
    p.sh = (int)sh; p.sw = (int)sw; p.ph = (int)ph; p.pw = (int)pw;
    p.PR = pl.PR; p.PW = pl.PW; p.L = (int)(OH * OW); p.tpi = pl.tpi; p.nchunks = pl.nchunks;
    p.div_tpi = FastDiv((uint32_t)pl.tpi);
    p.div_ow = FastDiv((uint32_t)OW);
    p.bt = (int)(B * pl.tpi);
    p.ntiles = (int)(B * pl.tpi * pl.mtiles);
    p.div_bt = FastDiv((uint32_t)p.bt);
    int nblk = std::min(p.ntiles, 2 * std::max(1, c->num_cus));  // two blocks per CU
    p.xcd_chunk = 0;
    if (p.ntiles % 8 == 0 && nblk >= 8) {
        nblk -= nblk % 8;
        p.xcd_chunk = p.ntiles / 8;
    }
    const dim3 grid((unsigned)nblk);
#define FX_CPD_LAUNCH(TNV)                                                                                             \
    case TNV: {                                                                                                        \
        static const hipError_t attr0 = hipFuncSetAttribute((const void*)conv_patch_f64_kernel<TNV, false>,            \
                                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_BYTES); \
        static const hipError_t attr1 = hipFuncSetAttribute((const void*)conv_patch_f64_kernel<TNV, true>,             \
                                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_BYTES); \
        FX_HIP_CHECK(attr0);                                                                                           \
        FX_HIP_CHECK(attr1);                                                                                           \
        if (bias) FX_LAUNCH(grid, dim3(NT), LDS_BYTES, c->stream, (p), conv_patch_f64_kernel<TNV, true>);                       \
        else FX_LAUNCH(grid, dim3(NT), LDS_BYTES, c->stream, (p), conv_patch_f64_kernel<TNV, false>);                           \
    } break;
    switch (pl.TN) {
        FX_CPD_LAUNCH(8)
        FX_CPD_LAUNCH(7)
        FX_CPD_LAUNCH(5)
        default: FX_REQUIRE(false, "conv patch kernel (f64): unexpected tile width %d", pl.TN);
    }
#undef FX_CPD_LAUNCH
    FX_LAUNCH_CHECK();
    return FX_OK;
}

}  // namespace cpd
