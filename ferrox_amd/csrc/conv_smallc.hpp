// 3x3 convolution over very few input channels (f32; an image layer: 1 to 4 channels forward, 1 to 3 for the weight
// gradient), the first layer of every network of the reference's examples (examples/common/models.rs:200-318; the
// product itself is conv2d_impl / cross_correlation2d_impl, src/backend/storage/extensions/convolutions.rs:218-338).
//
// With K = Cin*9 <= 36 the general kernels spend their time gathering a K x pixels operand whose rows are mostly
// padding of the 16-deep slabs.  Here a block copies the input rows under 256 consecutive output pixels of one image
// into LDS once, zero padded ([c][row][col]); the MFMA operand of lane l for reduction index k is then one LDS read at
// (pixel offset) + (tap offset of k), both cheap to form:
//   forward   y[oc][pixel] = sum_k w[oc][k] * patch(pixel, k)          A = w (registers, read in its natural [oc][c*9+t]
//             order, no re-layout pass), B = patch; one 32(oc) x 32(pixel) accumulator per 32 pixels, K/2 MFMAs each.
//   wgrad     dw[oc][k] = sum_pixel g[oc][pixel] * patch(pixel, k)     A = g staged as Gs[oc][pixel] (odd pitch),
//             B = patch with n = k; each wave reduces a quarter of the tile's pixels into one 32 x 32 accumulator, the
//             four are added through LDS at the end, blocks over disjoint pixel ranges leave partial sums that
//             the split-K reduction adds in order.  (Stride 1 / padding 1 layers take the row-band form further down.)
// Both are bound by the activation tensor they write / read (33.5 MB at [256,32,32,32]), not by the MFMA pipe.
#pragma once
#include "igemm_core.hpp"

namespace csc {
using igemm::FastDiv;
using igemm::f32x16;

constexpr int NT = 256, NPIX = 256, KK = 9;
constexpr int GP = NPIX + 1;                 // pitch of Gs: odd, so 32 output channels land on 32 banks
constexpr size_t LDS_LIMIT = 60 * 1024;

struct Geometry {
    int C, H, W, Cout, OH, OW, sh, sw, ph, pw;
    int PR, PW, PLANE;   // patch rows, padded row width, floats per channel plane
    int tpi;             // tiles of NPIX pixels per image
    FastDiv div_tpi, div_ow, div_w4, div_pr;
};

struct FwdParams {
    const float* x;
    const float* w;
    float* y;
    const float* bias;
    int relu;
    int ntiles;  // B * tiles per image
    Geometry g;
};

struct WgradParams {
    const float* x;
    const float* g;
    const float* act;    // MASK: the layer's ReLU output; g is used as g * (act > 0)
    float* part;
    float* bpart;        // MASK: per-split sums of the masked g over the split's pixels, [Cout] (the bias gradient)
    int stages, sps;     // B * tpi, stages per block
    i64 part_stride;     // floats between the partial sums of two splits (dw and bias alike)
    Geometry q;
};

// Copies the rows under tile `tile` of image b into the patch (rows outside the image become zero; the padding
// columns are zeroed by the caller once and never written).
__device__ __forceinline__ void stage_patch(const Geometry& g, const float* __restrict__ x, float* patch, int b, int iy0, int tid) {
    // ceil(W / 4) vectors per row; the last one is moved back to end with the row (overlapping its neighbour)
    const int W4 = (g.W + 3) >> 2, items = g.C * g.PR * W4;
    for (int i = tid; i < items; i += NT) {
        const int rc = (int)g.div_w4.div((uint32_t)i), q = min(4 * (i - rc * W4), g.W - 4);
        const int c = (int)g.div_pr.div((uint32_t)rc), r = rc - c * g.PR;
        const int iy = iy0 + r;
        const bool ok = iy >= 0 && iy < g.H;
        const float4 v = *reinterpret_cast<const float4*>(x + (((i64)b * g.C + c) * g.H + (ok ? iy : 0)) * g.W + q);
        float* d = patch + c * g.PLANE + r * g.PW + g.pw + q;
        d[0] = ok ? v.x : 0.f; d[1] = ok ? v.y : 0.f; d[2] = ok ? v.z : 0.f; d[3] = ok ? v.w : 0.f;
    }
}

// tap offset of reduction index k = c*9 + ky*3 + kx inside the patch (0 for the padding indices k >= K)
__device__ __forceinline__ int tap_offset(const Geometry& g, int k) {
    if (k >= g.C * KK) return 0;
    const int c = k / KK, t = k - c * KK, ky = t / 3, kx = t - ky * 3;
    return c * g.PLANE + ky * g.PW + kx;
}

// KS = ceil(Cin * 9 / 2) MFMA steps.  grid = (blocks, ceil(Cout / 32)); block x takes the (image, tile) pairs x, x + blocks, ...
// The patch of the next pair is loaded into registers before the MFMAs and stores of the current one (at most NPV float4 per
// thread), so a block's loads, MFMAs and stores overlap from its second tile on.
constexpr int NPV = 4;
template <int KS, bool BIAS>
__global__ __launch_bounds__(NT) void fwd_kernel(const FwdParams p) {
    FX_DYNAMIC_SMEM(float, patch);
    const Geometry& g = p.g;
    const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5, l32 = lane & 31;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int m0 = blockIdx.y * 32;
    const int L = g.OH * g.OW, K = g.C * KK;

    // the weight loads are in flight while the first patch is staged; they are first used after the second barrier
    float wraw[KS];
    int koff[KS];
    const bool m_ok = m0 + l32 < g.Cout;
    const float* wrow = p.w + (i64)(m_ok ? m0 + l32 : 0) * K;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        const int k = 2 * s + half;
        wraw[s] = wrow[k < K ? k : 0];
        koff[s] = tap_offset(g, k);
    }
    // per-thread constants of the staging: patch items tid + NT v (see stage_patch for the item -> (channel, row, vector) map)
    const int W4 = (g.W + 3) >> 2, items = g.C * g.PR * W4;
    int p_src[NPV], p_dst[NPV], p_row[NPV];
#pragma unroll
    for (int v = 0; v < NPV; ++v) {
        const int i = min(tid + v * NT, items - 1);
        const int rc = (int)g.div_w4.div((uint32_t)i), q = min(4 * (i - rc * W4), g.W - 4);
        const int c = (int)g.div_pr.div((uint32_t)rc), r = rc - c * g.PR;
        p_src[v] = c * g.H * g.W + q;
        p_dst[v] = c * g.PLANE + r * g.PW + g.pw + q;
        p_row[v] = r;
    }
    float4 pv[NPV];
    auto prefetch = [&](int t) __attribute__((always_inline)) {
        const int b = (int)g.div_tpi.div((uint32_t)t), tile = t - b * g.tpi;
        const int iy0 = (int)g.div_ow.div((uint32_t)(tile * NPIX)) * g.sh - g.ph;
#pragma unroll
        for (int v = 0; v < NPV; ++v) {
            if (v * NT >= items) break;  // block-uniform
            const int iy = iy0 + p_row[v];
            const bool ok = iy >= 0 && iy < g.H;
            pv[v] = *reinterpret_cast<const float4*>(p.x + (i64)b * g.C * g.H * g.W + p_src[v] + (ok ? iy : 0) * g.W);
            if (!ok) pv[v] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
    };
    // the bias of this lane's 16 output rows, loaded once (a load per tile in the store loop puts its latency on every tile)
    float bv[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) {
        const int ch = m0 + igemm::Mfma<float>::row(e, lane);
        bv[e] = BIAS ? p.bias[ch < g.Cout ? ch : g.Cout - 1] : 0.f;
    }
    const int ntiles = p.ntiles;
    int t = blockIdx.x;
    if (t < ntiles) prefetch(t);
    for (int i = tid; i < g.C * g.PLANE; i += NT) patch[i] = 0.f;  // the padding columns stay zero from here on
    float wreg[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) wreg[s] = m_ok && 2 * s + half < K ? wraw[s] : 0.f;

    for (; t < ntiles; t += gridDim.x) {
        const int b = (int)g.div_tpi.div((uint32_t)t), tile = t - b * g.tpi;
        const int pix0 = tile * NPIX, py0 = (int)g.div_ow.div((uint32_t)pix0);
        __syncthreads();  // the previous tile's reads are done (and the zero fill before the first)
#pragma unroll
        for (int v = 0; v < NPV; ++v) {
            if (v * NT >= items) break;
            if (tid + v * NT < items) {
                float* d = patch + p_dst[v];
                d[0] = pv[v].x; d[1] = pv[v].y; d[2] = pv[v].z; d[3] = pv[v].w;
            }
        }
        __syncthreads();
        if (t + (int)gridDim.x < ntiles) prefetch(t + gridDim.x);

        float* yb = p.y + (i64)b * g.Cout * L;
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
            const int pbase = pix0 + (wave * 2 + blk) * 32;
            if (pbase >= L) break;  // wave-uniform
            const int pp = pbase + l32, pc = min(pp, L - 1);
            const int oy = (int)g.div_ow.div((uint32_t)pc), ox = pc - oy * g.OW;
            const float* src = patch + (oy - py0) * g.sh * g.PW + ox * g.sw;
            f32x16 acc;
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[e] = 0.f;
#pragma unroll
            for (int s = 0; s < KS; ++s) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(wreg[s], src[koff[s]], acc, 0, 0, 0);
            if (pp < L) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int ch = m0 + igemm::Mfma<float>::row(e, lane);
                    if (ch < g.Cout) {
                        float v = acc[e];
                        if constexpr (BIAS) {
                            v += bv[e];
                            if (p.relu) v = v > 0.f ? v : 0.f;
                        }
                        yb[(i64)ch * L + pp] = v;
                    }
                }
            }
        }
    }
}

// grid = (splits, ceil(Cout / 32)); block z takes stages [z * sps, (z + 1) * sps), a stage being one tile of one image.
// Needs C * 9 <= 32 and (OH * OW) % 4 == 0.
// MASK: the gradient arrives unmasked from the layer above and the ReLU of this layer is applied while it is staged
// (g * (act > 0), the bits of fx_relu_bwd); reduction column K = C * 9 <= 27 of the 32 is free, and with a B operand of 1.0
// there the MFMA leaves sum over pixels of the masked g in it: the bias gradient, at no extra instruction.
template <bool MASK>
__global__ __launch_bounds__(NT, 2) void wgrad_kernel(const WgradParams p) {
    FX_DYNAMIC_SMEM(float, smem);
    const Geometry& g = p.q;
    float* Gs = smem;                 // [32][GP]
    float* patch = smem + 32 * GP;    // [C][PR][PW]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, l32 = lane & 31;
    const int m0 = blockIdx.y * 32, z = blockIdx.x;
    const int L = g.OH * g.OW, K = g.C * KK;
    const int toff = tap_offset(g, l32);
    const bool ones = MASK && l32 == K;
    f32x16 acc;
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = 0.f;
    for (int i = tid; i < g.C * g.PLANE; i += NT) patch[i] = 0.f;

    const int s_end = min(p.stages, (z + 1) * p.sps);
    const int gq = tid & 63, gr = tid >> 6;  // float4 column and first row of this thread in Gs
    for (int s = z * p.sps; s < s_end; ++s) {
        const int b = (int)g.div_tpi.div((uint32_t)s), tile = s - b * g.tpi;
        const int pix0 = tile * NPIX, py0 = (int)g.div_ow.div((uint32_t)pix0), iy0 = py0 * g.sh - g.ph;
        __syncthreads();  // the previous stage's reads are done (and the zero fill before the first)
        const bool col_ok = pix0 + 4 * gq < L;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int row = gr + 4 * u;
            const bool ok = col_ok && m0 + row < g.Cout;
            const i64 goff = ((i64)b * g.Cout + (ok ? m0 + row : 0)) * L + (ok ? pix0 + 4 * gq : 0);
            float4 v = *reinterpret_cast<const float4*>(p.g + goff);
            if constexpr (MASK) {
                const float4 a = *reinterpret_cast<const float4*>(p.act + goff);
                v.x = v.x * (a.x > 0.f ? 1.f : 0.f); v.y = v.y * (a.y > 0.f ? 1.f : 0.f);
                v.z = v.z * (a.z > 0.f ? 1.f : 0.f); v.w = v.w * (a.w > 0.f ? 1.f : 0.f);
            }
            float* d = Gs + row * GP + 4 * gq;
            d[0] = ok ? v.x : 0.f; d[1] = ok ? v.y : 0.f; d[2] = ok ? v.z : 0.f; d[3] = ok ? v.w : 0.f;
        }
        stage_patch(g, p.x, patch, b, iy0, tid);
        __syncthreads();
        const float* ga = Gs + l32 * GP + wave * 64 + half;
        const int pw0 = pix0 + wave * 64 + half;
#pragma unroll 4
        for (int st = 0; st < 32; ++st) {
            const int pc = min(pw0 + 2 * st, L - 1);  // past the end g is zero; the patch read only has to be in range
            const int oy = (int)g.div_ow.div((uint32_t)pc), ox = pc - oy * g.OW;
            float bv = patch[(oy - py0) * g.sh * g.PW + ox * g.sw + toff];
            if (MASK && ones) bv = 1.f;
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ga[2 * st], bv, acc, 0, 0, 0);
        }
    }
    // the four waves hold sums over different pixels: add them in wave order
    __syncthreads();
    float* red = smem;  // [4][16][64]
#pragma unroll
    for (int e = 0; e < 16; ++e) red[(wave * 16 + e) * 64 + lane] = acc[e];
    __syncthreads();
    float* out = p.part + (i64)z * p.part_stride;
    for (int i = tid; i < 16 * 64; i += NT) {
        const int e = i >> 6, ln = i & 63;
        const float v = ((red[i] + red[1024 + i]) + red[2048 + i]) + red[3072 + i];
        const int m = m0 + igemm::Mfma<float>::row(e, ln), n = ln & 31;
        if (m < g.Cout && n < K) out[(i64)m * K + n] = v;
        if (MASK && m < g.Cout && n == K) p.bpart[(i64)z * p.part_stride + m] = v;
    }
}

// ---- Row-band weight gradient: stride 1, padding 1 (output map = input map), rows of at most 64 floats that are a multiple of 4
// The tile kernel above stages g through LDS behind two block barriers per tile, and its blocks run in lockstep on a layer of
// this size.  Here every WAVE is on its own: it takes a band of `rb` output rows of one image, copies the rb + 2 input rows under
// it into its private piece of LDS, and feeds g to the MFMA straight from global memory, two steps of loads in flight, without
// meeting a block barrier before the closing sum.  [256,3,32,32] -> 32: 20.2 -> 13.5 us, with the ReLU mask and the bias sums
// 25.3 -> 18.3 us (kernel + ordered sum).  (The same scheme for the forward pass measured level with the tile kernel, 15.2 against
// 15.9 us with bias and ReLU: its time is the sum of launch, first loads, MFMAs and the 33.5 MB of stores either way.)
struct RowGeometry {
    int C, H, W, Cout, B;
    int rb, bands;      // output rows per band, bands per image
    int cbs;            // blocks of 32 pixels per row
    int PW, PLANE;      // padded row width W + 2, floats per channel plane (rb + 2) * PW
    int wave_floats;    // floats of LDS per wave: C * PLANE + slack for the reads past a short row's end
    int ntasks;         // B * bands
    FastDiv div_bands, div_w4, div_pr;
};
struct RowWgradParams {
    const float* x;
    const float* g;
    const float* act;
    float* part;
    float* bpart;
    i64 part_stride;
    RowGeometry q;
};
constexpr int ROW_NPV = 4;      // float4 of the patch one lane keeps in flight: C * (rb + 2) * W / 4 <= 4 * 64
constexpr int ROW_SLACK = 36;   // floats behind a wave's planes that a read past a short row's end may touch

// The rows [oy0 - 1, oy0 + rb] of image b into this wave's patch, zero above and below the image; columns 0 and W + 1 of every
// row are the zero padding (written here as well: the patch is private to the wave and nothing else clears it).
__device__ __forceinline__ void stage_band(const RowGeometry& q, const float* __restrict__ x, float* patch, int b, int oy0, int lane) {
    const int W4 = q.W >> 2, PR = q.rb + 2, items = q.C * PR * W4;
    float4 v[ROW_NPV];
    int dst[ROW_NPV];
#pragma unroll
    for (int u = 0; u < ROW_NPV; ++u) {
        const int i = min(lane + 64 * u, items - 1);
        const int rc = (int)q.div_w4.div((uint32_t)i), col = 4 * (i - rc * W4);
        const int c = (int)q.div_pr.div((uint32_t)rc), r = rc - c * PR;
        const int iy = oy0 - 1 + r;
        const bool ok = iy >= 0 && iy < q.H;
        v[u] = *reinterpret_cast<const float4*>(x + (((i64)b * q.C + c) * q.H + (ok ? iy : 0)) * q.W + col);
        if (!ok) v[u] = make_float4(0.f, 0.f, 0.f, 0.f);
        dst[u] = c * q.PLANE + r * q.PW + 1 + col;
    }
    for (int i = lane; i < q.C * PR; i += 64) {
        patch[i * q.PW] = 0.f;
        patch[i * q.PW + q.W + 1] = 0.f;
    }
    if (lane < ROW_SLACK) patch[q.C * q.PLANE + lane] = 0.f;  // what a read past a short row's end finds there is multiplied by a zero of g
#pragma unroll
    for (int u = 0; u < ROW_NPV; ++u)
        if (lane + 64 * u < items) {
            float* d = patch + dst[u];
            d[0] = v[u].x; d[1] = v[u].y; d[2] = v[u].z; d[3] = v[u].w;
        }
    __builtin_amdgcn_wave_barrier();  // one wave: its LDS accesses complete in program order, so this is a scheduling fence only
}

__device__ __forceinline__ int row_tap_offset(const RowGeometry& q, int k) {
    if (k >= q.C * KK) return 0;
    const int c = k / KK, t = k - c * KK, ky = t / 3, kx = t - ky * 3;
    return c * q.PLANE + ky * q.PW + kx;
}

// grid = (ceil(tasks / 4), ceil(Cout / 32)).  Lane (oc = l % 32, h = l / 32) feeds the MFMA the 16 pixels 16 h .. 16 h + 15 of a
// block of 32 pixels of a row, straight from global memory (four 16-byte loads; the reduction index of the MFMA is a pixel, and
// which pixel goes to which step is free as long as both operands agree), the patch values of the same pixels from the wave's
// LDS.  A wave adds its whole band into one 32 x 32 accumulator; the four waves of a block are added through LDS in wave order and
// the block leaves one partial sum, which the ordered reduction adds over the blocks.
// MASK and the bias sums: as in wgrad_kernel above.
template <bool MASK>
__global__ __launch_bounds__(NT) void wgrad_rows_kernel(const RowWgradParams p) {
    FX_DYNAMIC_SMEM(float, smem);
    const RowGeometry& q = p.q;
    const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5, l32 = lane & 31;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int task = blockIdx.x * 4 + wave;
    float* patch = smem + wave * q.wave_floats;
    const int m0 = blockIdx.y * 32, K = q.C * KK;
    const int toff = row_tap_offset(q, l32);
    const bool ones = MASK && l32 == K;
    f32x16 acc;
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = 0.f;
    if (task < q.ntasks) {  // wave-uniform
        const int b = (int)q.div_bands.div((uint32_t)task), oy0 = (task - b * q.bands) * q.rb;
        const int nr = min(q.rb, q.H - oy0);
        const bool m_ok = m0 + l32 < q.Cout;
        const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
        const i64 grow = (((i64)b * q.Cout + (m_ok ? m0 + l32 : 0)) * q.H + oy0) * q.W;
        const int steps = nr * q.cbs;
        float4 gv[2][4], av[2][4];
        auto load = [&](int set, int st) __attribute__((always_inline)) {
            const int r = st / q.cbs, cb = st - r * q.cbs;
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int col = cb * 32 + half * 16 + 4 * u;
                const bool ok = m_ok && col < q.W;  // W is a multiple of 4: a vector is inside the row or past it
                const i64 off = grow + (i64)r * q.W + (ok ? col : 0);
                gv[set][u] = *reinterpret_cast<const float4*>(p.g + off);
                if (!ok) gv[set][u] = zero4;
                if constexpr (MASK) av[set][u] = *reinterpret_cast<const float4*>(p.act + off);
            }
        };
        auto mul = [&](int set, int st) __attribute__((always_inline)) {
            const int r = st / q.cbs, cb = st - r * q.cbs;
            const float* src = patch + r * q.PW + cb * 32 + half * 16 + toff;
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                float4 v = gv[set][u];
                if constexpr (MASK) {
                    const float4 a = av[set][u];
                    v.x = v.x * (a.x > 0.f ? 1.f : 0.f); v.y = v.y * (a.y > 0.f ? 1.f : 0.f);
                    v.z = v.z * (a.z > 0.f ? 1.f : 0.f); v.w = v.w * (a.w > 0.f ? 1.f : 0.f);
                }
                const float ge[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    float bvv = src[4 * u + j];
                    if (MASK && ones) bvv = 1.f;
                    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ge[j], bvv, acc, 0, 0, 0);
                }
            }
        };
        load(0, 0);
        stage_band(q, p.x, patch, b, oy0, lane);
        for (int st = 0; st < steps; st += 2) {
            if (st + 1 < steps) load(1, st + 1);
            mul(0, st);
            if (st + 2 < steps) load(0, st + 2);
            if (st + 1 < steps) mul(1, st + 1);
        }
    }
    // the four waves hold sums over different bands: add them in wave order (the patches are dead after the barrier)
    __syncthreads();
    float* red = smem;  // [4][16][64]
#pragma unroll
    for (int e = 0; e < 16; ++e) red[(wave * 16 + e) * 64 + lane] = acc[e];
    __syncthreads();
    float* out = p.part + (i64)blockIdx.x * p.part_stride;
    for (int i = tid; i < 16 * 64; i += NT) {
        const int e = i >> 6, ln = i & 63;
        const float v = ((red[i] + red[1024 + i]) + red[2048 + i]) + red[3072 + i];
        const int m = m0 + igemm::Mfma<float>::row(e, ln), n = ln & 31;
        if (m < q.Cout && n < K) out[(i64)m * K + n] = v;
        if (MASK && m < q.Cout && n == K) p.bpart[(i64)blockIdx.x * p.part_stride + m] = v;
    }
}

struct Plan {
    bool ok = false;
    int PR = 0, PW = 0, PLANE = 0, tpi = 0;
    int splits = 1, sps = 1, stages = 0;  // weight gradient only
    size_t smem = 0;
    int rb = 0;   // > 0: the row-band weight-gradient kernel with bands of rb output rows (splits = its blocks); 0: the tile kernels
    i64 B = 0;
};

inline Plan make_plan(int num_cus, bool wgrad, i64 B, i64 C, i64 H, i64 W, i64 Cout, i64 kh, i64 kw, i64 sh, i64 sw, i64 ph, i64 pw,
                      i64 OH, i64 OW) {
    Plan pl;
    const i64 L = OH * OW;
    if (kh != 3 || kw != 3 || W < 4 || sh > 8 || sw > 8 || ph > 8 || pw > 8) return pl;
    if (wgrad ? (C * KK > 32 || L % 4 != 0) : C > 4) return pl;
    pl.B = B;
    // Row-band weight gradient: output map = input map, rows of at most 64 floats.  Band height: about one wave per SIMD (measured
    // at [256,3,32,32] -> 32: 23.0 / 16.6 / 15.4 / 13.5 us with bands of 1 / 2 / 4 / 8 rows; at [32,1,28,28] -> 8 bands of 2 are the
    // fastest), within what one lane stages (ROW_NPV vectors).
    if (wgrad && sh == 1 && sw == 1 && ph == 1 && pw == 1 && OH == H && OW == W && W % 4 == 0 && W <= 64 && B * H <= 0x3fffffff) {
        i64 rb = std::max<i64>(2, std::min<i64>(8, B * H / (4 * (i64)std::max(1, num_cus))));
        rb = std::min<i64>(rb, H);
        while (rb > 1 && C * (rb + 2) * (W / 4) > ROW_NPV * 64) --rb;
        if (C * (rb + 2) * (W / 4) <= ROW_NPV * 64 && fx::ceil_div(Cout, (i64)32) <= 65535) {
            pl.rb = (int)rb;
            pl.PW = (int)(W + 2);
            pl.PLANE = (int)((rb + 2) * (W + 2));
            const i64 tasks = B * fx::ceil_div(H, rb);
            pl.splits = (int)fx::ceil_div(tasks, (i64)4);
            pl.stages = (int)tasks;
            pl.smem = std::max<size_t>((size_t)4 * (C * pl.PLANE + ROW_SLACK) * sizeof(float), 4 * 16 * 64 * sizeof(float));
            pl.ok = true;
            return pl;
        }
    }
    const i64 rows = std::min<i64>(OH, NPIX % OW == 0 ? NPIX / OW : (NPIX - 1) / OW + 2);
    pl.PR = (int)((rows - 1) * sh + 3);
    // wide images: a tile of 256 pixels covers about one output row and would stage five or seven input rows (measured
    // at 3 x 224 x 224 -> 64: 0.300 ms here against 0.245 ms for the implicit GEMM, 0.074 against 0.059 ms at stride 2)
    // (rows up to 256 floats that divide the tile -- 128: two rows per tile -- stage four rows for two and stay ahead of it)
    if ((OW > 64 && (OW > NPIX || NPIX % OW != 0)) || (i64)pl.PR * OW > 2 * (i64)NPIX * sh) return pl;
    pl.PW = (int)(W + 2 * pw);
    pl.PLANE = pl.PR * pl.PW;
    pl.tpi = (int)fx::ceil_div(L, (i64)NPIX);
    pl.smem = ((size_t)C * pl.PLANE + (wgrad ? (size_t)32 * GP : 0)) * sizeof(float);
    if (pl.smem > LDS_LIMIT || B * pl.tpi > 0x7fffffff) return pl;
    if (!wgrad && C * pl.PR * ((W + 3) / 4) > NPV * NT) return pl;  // the patch items one thread keeps in flight
    if (wgrad) {
        pl.stages = (int)(B * pl.tpi);
        const i64 mblocks = fx::ceil_div(Cout, (i64)32);
        const i64 splits = std::max<i64>(1, std::min<i64>(pl.stages, 4 * (i64)num_cus / mblocks));
        pl.sps = (int)fx::ceil_div((i64)pl.stages, splits);
        pl.splits = (int)fx::ceil_div((i64)pl.stages, (i64)pl.sps);
        if (mblocks > 65535) return pl;
    } else if (fx::ceil_div(Cout, (i64)32) > 65535) {
        return pl;
    }
    pl.ok = true;
    return pl;
}

// the masked variant keeps [Cout] bias sums behind every split's [Cout][C*9] partial
inline i64 wgrad_workspace_bytes(const Plan& pl, i64 Cout, i64 C, bool with_bias = false) {
    return pl.splits > 1 ? (i64)pl.splits * (Cout * C * KK + (with_bias ? Cout : 0)) * (i64)sizeof(float) : 0;
}

inline Geometry make_geometry(const Plan& pl, i64 C, i64 H, i64 W, i64 Cout, i64 OH, i64 OW, i64 sh, i64 sw, i64 ph, i64 pw) {
    Geometry g;
    g.C = (int)C; g.H = (int)H; g.W = (int)W; g.Cout = (int)Cout; g.OH = (int)OH; g.OW = (int)OW;
    g.sh = (int)sh; g.sw = (int)sw; g.ph = (int)ph; g.pw = (int)pw;
    g.PR = pl.PR; g.PW = pl.PW; g.PLANE = pl.PLANE; g.tpi = pl.tpi;
    g.div_tpi = FastDiv((uint32_t)pl.tpi); g.div_ow = FastDiv((uint32_t)OW);
    g.div_w4 = FastDiv((uint32_t)((W + 3) / 4)); g.div_pr = FastDiv((uint32_t)pl.PR);
    return g;
}

// x and y's base addresses must be 16-byte aligned (x for the vector loads).
inline RowGeometry make_row_geometry(const Plan& pl, i64 B, i64 C, i64 H, i64 W, i64 Cout) {
    RowGeometry q;
    q.C = (int)C; q.H = (int)H; q.W = (int)W; q.Cout = (int)Cout; q.B = (int)B;
    q.rb = pl.rb; q.bands = (int)fx::ceil_div(H, (i64)pl.rb); q.cbs = (int)fx::ceil_div(W, (i64)32);
    q.PW = pl.PW; q.PLANE = pl.PLANE; q.wave_floats = (int)(C * pl.PLANE + ROW_SLACK);
    q.ntasks = (int)(B * q.bands);
    q.div_bands = FastDiv((uint32_t)q.bands); q.div_w4 = FastDiv((uint32_t)(W / 4)); q.div_pr = FastDiv((uint32_t)(pl.rb + 2));
    return q;
}

inline int run_fwd(fx_ctx* c, const Plan& pl, const float* x, const float* w, float* y, i64 B, i64 C, i64 H, i64 W, i64 Cout, i64 OH,
                   i64 OW, i64 sh, i64 sw, i64 ph, i64 pw, const float* bias, int relu) {
    FwdParams p;
    p.x = x; p.w = w; p.y = y; p.bias = bias; p.relu = relu;
    p.g = make_geometry(pl, C, H, W, Cout, OH, OW, sh, sw, ph, pw);
    p.ntiles = (int)(B * pl.tpi);
    // two blocks per CU for every row of 32 output channels, every block with the same number of tiles (measured at
    // [256,3,32,32]: -> 32 13.9 us one tile per block, 14.0 / 12.7 / 13.6 us at one / two / four blocks per CU; -> 64 20.9 one tile
    // per block, 21.2 / 20.7 at two / four blocks per CU over both rows)
    const i64 mblocks = fx::ceil_div(Cout, (i64)32);
    const i64 want = std::max<i64>(1, 2 * (i64)c->num_cus);
    const i64 per_block = fx::ceil_div((i64)p.ntiles, want);
    const dim3 grid((unsigned)fx::ceil_div((i64)p.ntiles, per_block), (unsigned)mblocks);
#define FX_CSC_FWD(KSV)                                                                                 \
    do {                                                                                                \
        if (bias) FX_LAUNCH(grid, dim3(NT), pl.smem, c->stream, (p), fwd_kernel<KSV, true>);                     \
        else FX_LAUNCH(grid, dim3(NT), pl.smem, c->stream, (p), fwd_kernel<KSV, false>);                         \
    } while (0)
    switch ((int)C) {
        case 1: FX_CSC_FWD(5); break;
        case 2: FX_CSC_FWD(9); break;
        case 3: FX_CSC_FWD(14); break;
        default: FX_CSC_FWD(18); break;
    }
#undef FX_CSC_FWD
    FX_LAUNCH_CHECK();
    return FX_OK;
}

// x, g and part 16-byte aligned.  part holds splits x [Cout][C*9] partial sums (unused when splits == 1).
// act / db non-null: the masked variant (g * (act > 0) staged, db = its sums per output channel), act 16-byte aligned too.
inline int run_wgrad(fx_ctx* c, const Plan& pl, const float* x, const float* g, float* dw, float* part, i64 C, i64 H, i64 W, i64 Cout,
                     i64 OH, i64 OW, i64 sh, i64 sw, i64 ph, i64 pw, const float* act = nullptr, float* db = nullptr) {
    const i64 n = Cout * C * KK;
    if (pl.rb) {
        RowWgradParams rp;
        rp.x = x; rp.g = g; rp.act = act;
        rp.part = pl.splits > 1 ? part : dw;
        rp.bpart = pl.splits > 1 ? part + n : db;
        rp.part_stride = n + (act ? Cout : 0);
        rp.q = make_row_geometry(pl, pl.B, C, H, W, Cout);
        const dim3 grid((unsigned)pl.splits, (unsigned)fx::ceil_div(Cout, (i64)32));
        if (act) FX_LAUNCH(grid, dim3(NT), pl.smem, c->stream, (rp), wgrad_rows_kernel<true>);
        else FX_LAUNCH(grid, dim3(NT), pl.smem, c->stream, (rp), wgrad_rows_kernel<false>);
        FX_LAUNCH_CHECK();
        if (pl.splits > 1) {
            if (act) return igemm::launch_splitk_reduce_pair<float>(c, part, rp.part_stride, pl.splits, dw, n, db, Cout);
            return igemm::launch_splitk_reduce<float>(c, part, dw, n, pl.splits);
        }
        return FX_OK;
    }
    WgradParams p;
    p.x = x; p.g = g; p.act = act;
    p.part = pl.splits > 1 ? part : dw;
    p.bpart = pl.splits > 1 ? part + n : db;
    p.stages = pl.stages; p.sps = pl.sps; p.part_stride = n + (act ? Cout : 0);
    p.q = make_geometry(pl, C, H, W, Cout, OH, OW, sh, sw, ph, pw);
    const dim3 grid((unsigned)pl.splits, (unsigned)fx::ceil_div(Cout, (i64)32));
    if (act) FX_LAUNCH(grid, dim3(NT), pl.smem, c->stream, (p), wgrad_kernel<true>);
    else FX_LAUNCH(grid, dim3(NT), pl.smem, c->stream, (p), wgrad_kernel<false>);
    FX_LAUNCH_CHECK();
    if (pl.splits > 1) {
        if (act) return igemm::launch_splitk_reduce_pair<float>(c, part, p.part_stride, pl.splits, dw, n, db, Cout);
        return igemm::launch_splitk_reduce<float>(c, part, dw, n, pl.splits);
    }
    return FX_OK;
}

}  // namespace csc
