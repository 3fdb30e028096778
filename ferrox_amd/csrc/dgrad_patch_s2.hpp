// Data gradient of a 3x3 convolution of stride 2 and padding 1 over an even-sized map (f32):
//   dx[b][c][iy][ix] = sum over (oc, ky, kx) with iy + 1 - ky = 2 oy, ix + 1 - kx = 2 ox of g[b][oc][oy][ox] * w[oc][c][ky][kx]
// (col2im(W2d^T . grad_out) in the reference, src/backend/storage/extensions/convolutions.rs:268-294).
//
// The input pixels of grid cell (i, j) -- (2i + py, 2j + px), py, px in {0, 1} -- receive only the taps of their parity class,
// and all of them from the four grad_out pixels (i, j), (i, j+1), (i+1, j), (i+1, j+1):
//   (0,0): w11 g(i,j)                 (0,1): w10 g(i,j+1) + w12 g(i,j)                 (1,0): w01 g(i+1,j) + w21 g(i,j)
//   (1,1): w00 g(i+1,j+1) + w02 g(i+1,j) + w20 g(i,j+1) + w22 g(i,j)
// so the nine taps run exactly once per cell (the all-taps gather would multiply 3 zeros in 4), and the four classes share
// their operand reads.  A block (8 waves) takes 256 cells of one image -- TR = 256 / OW grid rows -- and 32 input channels;
// a wave owns 32 cells and keeps one 32(c) x 32(cell) accumulator block per class.  The output channels are reduced in chunks
// of OCC; per chunk the block holds in LDS
//   Ws[oc pair][tap][lane]    the MFMA A operand as the lanes read it: lane l holds w[oc = 2 pair + l / 32][c = l % 32][tap]
//   Gs[oc][row][col]          the (TR + 1) x (OW + 1) patch of grad_out (row TR is the next tile's first row or zero, column OW
//                             is zero), odd plane pitch
// in two buffers: the next chunk is loaded into registers before the MFMA loop of the current one and parked after it, a chunk
// costs one barrier.  Per oc pair a wave reads 9 weights and 4 patch values for its 9 MFMAs, all at immediate offsets.  The
// two column classes of a cell are stored together as one 8-byte pair, so a half-wave writes whole 128-byte rows of dx.
#pragma once
#include <cstdlib>

#include "igemm_core.hpp"

namespace dg2 {
using igemm::FastDiv;
using igemm::f32x16;
using igemm::ldg4;

constexpr int KK = 9, NT = 512, CT = 32, CELLS = 256;
constexpr size_t LDS_LIMIT = 160 * 1024;

struct Params {
    const float* g;
    const float* act;  // MASK: the ReLU output of the layer whose gradient g is; g is staged as g * (act > 0)
    const float* w;
    float* dx;
    int Cin, Cout, oh, tpi, nct;  // tiles per image, channel tiles
    FastDiv div_nct, div_tpi;
};

template <int OW, int OCC>
struct Shape {
    static constexpr int TR = CELLS / OW, PC = OW + 1, PR = TR + 1;
    static constexpr int GPL = (PR * PC) | 1;              // plane pitch of the patch
    static constexpr int KS = OCC / 2;                     // MFMA steps (oc pairs) per chunk
    static constexpr int WCH = KS * KK * 64, GCH = OCC * GPL, BUF = WCH + GCH;
    static constexpr size_t LDS = 2 * (size_t)BUF * sizeof(float);
    static constexpr int W4 = OCC * CT * KK / 4;           // float4 of a weight chunk (32 x 9 contiguous floats per oc)
    static constexpr int NWP = (W4 + NT - 1) / NT;         // passes over them
    static constexpr int NGP = OCC * (CELLS / 4) / NT;     // passes over the TR full rows of the patch (64 float4 per oc)
    static constexpr int X4 = OCC * OW / 4;                // float4 of the extra row
    static_assert(CELLS % OW == 0 && OW % 4 == 0 && OCC % 8 == 0 && OCC * (CELLS / 4) % NT == 0 && X4 <= NT && LDS <= LDS_LIMIT, "shape");
};

// MASK: grad_out arrives unmasked and the layer's ReLU is applied to the staged patch (g * (act > 0), the bits of fx_relu_bwd).
template <int OW, int OCC, bool MASK>
__global__ __launch_bounds__(NT, 1) void dgrad_s2_kernel(const Params p) {
    using S = Shape<OW, OCC>;
    constexpr int TR = S::TR, PC = S::PC, GPL = S::GPL, KS = S::KS, WCH = S::WCH, BUF = S::BUF;
    FX_DYNAMIC_SMEM(float, smem);
    const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5, l32 = lane & 31;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int bt = (int)p.div_nct.div(blockIdx.x), ct = (int)blockIdx.x - bt * p.nct;
    const int b = (int)p.div_tpi.div((uint32_t)bt), tile = bt - b * p.tpi;
    const int c0 = ct * CT, i0 = tile * TR;
    const int L = p.oh * OW, H = 2 * p.oh, W = 2 * OW;
    const bool next_row = i0 + TR < p.oh;  // the patch's last row exists in grad_out (block-uniform)

    // staging maps (constant over the chunks)
    const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
    float4 wv[S::NWP], gv[S::NGP], xv, av[MASK ? S::NGP : 1], axv;
    const float* wsrc = p.w + (i64)c0 * KK;
    const float* gsrc = p.g + ((i64)b * p.Cout * p.oh + i0) * OW;
    const float* asrc = MASK ? p.act + ((i64)b * p.Cout * p.oh + i0) * OW : nullptr;
    auto masked = [](float4 v, const float4& a) __attribute__((always_inline)) {
        v.x = v.x * (a.x > 0.f ? 1.f : 0.f); v.y = v.y * (a.y > 0.f ? 1.f : 0.f);
        v.z = v.z * (a.z > 0.f ? 1.f : 0.f); v.w = v.w * (a.w > 0.f ? 1.f : 0.f);
        return v;
    };
    const int gq = tid & 63, goc = tid >> 6;                    // float4 of the tile's TR * OW floats, oc within a pass of 8
    const int g_dst = goc * GPL + (gq / (OW / 4)) * PC + (gq % (OW / 4)) * 4;
    const uint32_t g_off = (uint32_t)(goc * L + 4 * gq) * 4u;
    const int xoc = tid / (OW / 4), xq = tid % (OW / 4);        // extra row: oc, float4 column
    const bool x_lane = tid < S::X4;
    const uint32_t x_off = x_lane ? (uint32_t)(xoc * L + TR * OW + 4 * xq) * 4u : 0u;
    auto prefetch = [&](int k) __attribute__((always_inline)) {
        const int oc0 = k * OCC;
#pragma unroll
        for (int u = 0; u < S::NWP; ++u) {
            const int f = u * NT + tid;
            const bool ok = (u + 1) * NT <= S::W4 || f < S::W4;
            const int ocl = f / 72, q = f - ocl * 72;
            wv[u] = ldg4(wsrc + (i64)oc0 * p.Cin * KK, ok ? (uint32_t)(ocl * p.Cin * KK + 4 * q) * 4u : 0u);
        }
#pragma unroll
        for (int u = 0; u < S::NGP; ++u) gv[u] = ldg4(gsrc + (i64)(oc0 + 8 * u) * L, g_off);
        if (next_row) xv = ldg4(gsrc + (i64)oc0 * L, x_off);
        else xv = zero4;
        if constexpr (MASK) {
#pragma unroll
            for (int u = 0; u < S::NGP; ++u) av[u] = ldg4(asrc + (i64)(oc0 + 8 * u) * L, g_off);
            if (next_row) axv = ldg4(asrc + (i64)oc0 * L, x_off);
            else axv = zero4;
        }
    };
    auto park = [&](int buf) __attribute__((always_inline)) {
        float* Ws = smem + buf * BUF;
        float* Gs = Ws + WCH;
#pragma unroll
        for (int u = 0; u < S::NWP; ++u) {
            const int f = u * NT + tid;
            if ((u + 1) * NT <= S::W4 || f < S::W4) {
                const int ocl = f / 72, q = f - ocl * 72;
                const float v[4] = {wv[u].x, wv[u].y, wv[u].z, wv[u].w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int e = 4 * q + i, c = e / KK, t = e - c * KK;
                    Ws[((ocl >> 1) * KK + t) * 64 + (ocl & 1) * 32 + c] = v[i];
                }
            }
        }
#pragma unroll
        for (int u = 0; u < S::NGP; ++u) {
            float* d = Gs + g_dst + 8 * u * GPL;
            if constexpr (MASK) gv[u] = masked(gv[u], av[u]);
            d[0] = gv[u].x; d[1] = gv[u].y; d[2] = gv[u].z; d[3] = gv[u].w;
        }
        if (x_lane) {
            float* d = Gs + xoc * GPL + TR * PC + 4 * xq;
            if constexpr (MASK) xv = masked(xv, axv);
            d[0] = xv.x; d[1] = xv.y; d[2] = xv.z; d[3] = xv.w;
        }
    };

    f32x16 acc[2][2];  // [py][px]
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int q = 0; q < 2; ++q)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[a][q][e] = 0.f;

    // this wave's cells: wave * 32 + l32 of the tile, row-major; lane l reads the patch plane of oc = 2 pair + l / 32
    const int cell = wave * 32 + l32, crow = cell / OW, ccol = cell % OW;
    const int gb0 = WCH + half * GPL + crow * PC + ccol;
    auto compute = [&](int buf) __attribute__((always_inline)) {
        const float* wa = smem + buf * BUF + lane;
        const float* gb = smem + buf * BUF + gb0;
        float a[KS][KK], bq[KS][4];
        auto rd = [&](int ks) __attribute__((always_inline)) {
#pragma unroll
            for (int t = 0; t < KK; ++t) a[ks][t] = wa[(ks * KK + t) * 64];
            bq[ks][0] = gb[2 * ks * GPL];
            bq[ks][1] = gb[2 * ks * GPL + 1];
            bq[ks][2] = gb[2 * ks * GPL + PC];
            bq[ks][3] = gb[2 * ks * GPL + PC + 1];
            __builtin_amdgcn_sched_barrier(0);
        };
        rd(0);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            if (ks + 1 < KS) rd(ks + 1);
            // taps w[ky][kx] = a[3 ky + kx]; b: 0 = g(i,j), 1 = g(i,j+1), 2 = g(i+1,j), 3 = g(i+1,j+1).  The four products of class
            // (1,1) alternate with the others so that no MFMA waits for the one before it.
            acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[ks][0], bq[ks][3], acc[1][1], 0, 0, 0);
            acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[ks][4], bq[ks][0], acc[0][0], 0, 0, 0);
            acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[ks][2], bq[ks][2], acc[1][1], 0, 0, 0);
            acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[ks][3], bq[ks][1], acc[0][1], 0, 0, 0);
            acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[ks][6], bq[ks][1], acc[1][1], 0, 0, 0);
            acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[ks][1], bq[ks][2], acc[1][0], 0, 0, 0);
            acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[ks][8], bq[ks][0], acc[1][1], 0, 0, 0);
            acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[ks][5], bq[ks][0], acc[0][1], 0, 0, 0);
            acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[ks][7], bq[ks][0], acc[1][0], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    const int nchunks = p.Cout / OCC;
    prefetch(0);
    // column OW of every patch row is the zero padding right of the map: written once in both buffers
    for (int i = tid; i < 2 * OCC * S::PR; i += NT) {
        const int buf = i / (OCC * S::PR), rem = i - buf * (OCC * S::PR), oc = rem / S::PR, r = rem - oc * S::PR;
        smem[buf * BUF + WCH + oc * GPL + r * PC + OW] = 0.f;
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
    float* out = p.dx + (((i64)b * p.Cin + c0) * H + 2 * (i0 + crow)) * W + 2 * ccol;
#pragma unroll
    for (int py = 0; py < 2; ++py)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const int c = igemm::Mfma<float>::row(e, lane);
            *reinterpret_cast<float2*>(out + ((i64)c * H + py) * W) = make_float2(acc[py][0][e], acc[py][1][e]);
        }
}

struct Plan {
    bool ok = false;
    int OW = 0, OCC = 0;
    size_t smem = 0;
};

// Instantiated (OW, OCC): maps 32 and 64 wide.  Chunks of 16 output channels measured level with chunks of 32 (29.2 against
// 29.8 us at [256,32,32,32] <- 64) at half the LDS.
#define FX_DG2_SHAPES(X) X(16, 16) X(32, 16)

inline Plan make_plan(i64 B, i64 Cin, i64 H, i64 W, i64 Cout, i64 kh, i64 kw, i64 sh, i64 sw, i64 ph, i64 pw, i64 oh, i64 ow) {
    Plan pl;
    if (kh != 3 || kw != 3 || sh != 2 || sw != 2 || ph != 1 || pw != 1 || W != 2 * ow || H != 2 * oh || Cin % CT != 0) return pl;
    if (Cout * oh * ow * 4 > 0x7fffffff || Cout * Cin * KK * 4 > 0x7fffffff || B * (Cin / CT) * oh > 0x7fffffff) return pl;
#define FX_DG2_PICK(O, C_)                                                                   \
    if (!pl.ok && ow == O && Cout % C_ == 0 && oh % (CELLS / O) == 0) {                      \
        pl.ok = true; pl.OW = O; pl.OCC = C_; pl.smem = Shape<O, C_>::LDS;                   \
    }
    FX_DG2_SHAPES(FX_DG2_PICK)
#undef FX_DG2_PICK
    return pl;
}

// g, w and dx must be 16-byte aligned (dx for its 8-byte pairs).
// act non-null: the masked variant (act 16-byte aligned as well).
inline int run(fx_ctx* c, const Plan& pl, const float* g, const float* w, float* dx, i64 B, i64 Cin, i64 Cout, i64 oh,
               const float* act = nullptr) {
    Params p;
    p.g = g; p.w = w; p.dx = dx; p.act = act;
    p.Cin = (int)Cin; p.Cout = (int)Cout; p.oh = (int)oh;
    p.tpi = (int)(oh / (CELLS / pl.OW));
    p.nct = (int)(Cin / CT);
    p.div_nct = FastDiv((uint32_t)p.nct);
    p.div_tpi = FastDiv((uint32_t)p.tpi);
    const dim3 grid((unsigned)(B * p.tpi * p.nct));
    bool launched = false;
#define FX_DG2_LAUNCH(O, C_)                                                                                           \
    if (!launched && pl.OW == O && pl.OCC == C_) {                                                                     \
        static const hipError_t attr = hipFuncSetAttribute((const void*)dgrad_s2_kernel<O, C_, false>,                 \
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_LIMIT); \
        static const hipError_t attr_m = hipFuncSetAttribute((const void*)dgrad_s2_kernel<O, C_, true>,                \
                                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_LIMIT); \
        FX_HIP_CHECK(attr);                                                                                            \
        FX_HIP_CHECK(attr_m);                                                                                          \
        if (act) FX_LAUNCH(grid, dim3(NT), pl.smem, c->stream, (p), dgrad_s2_kernel<O, C_, true>);                              \
        else FX_LAUNCH(grid, dim3(NT), pl.smem, c->stream, (p), dgrad_s2_kernel<O, C_, false>);                                 \
        launched = true;                                                                                               \
    }
    FX_DG2_SHAPES(FX_DG2_LAUNCH)
#undef FX_DG2_LAUNCH
    FX_REQUIRE(launched, "dgrad stride-2 patch kernel: unexpected shape (%d, %d)", pl.OW, pl.OCC);
    FX_LAUNCH_CHECK();
    return FX_OK;
}

}  // namespace dg2
