// Weight gradient of a 3x3 convolution (f32) with both operands staged in LDS in their natural layouts.
//
// dw[oc][c][ky][kx] = sum over (b, oy, ox) of g[b][oc][oy][ox] * x[b][c][oy*sh+ky-ph][ox*sw+kx-pw]
// (the product the reference forms as grad_out_2d . im2col(x)^T, src/backend/storage/extensions/convolutions.rs:296-338).
//
// One stage = R output rows of one image.  A block (4 waves) copies, per stage,
//   Gs[oc][pixel]      BM output-channel rows of g, pixels contiguous as in memory  (pitch GP,    GP % 32 == 1)
//   Xs[c][row][col]    CT input-channel planes of the zero-padded rows those pixels touch (pitch PLANE % 32 == 1)
// The four waves are laid out WMO x WC x WK: WMO blocks of 32 output channels (BM = 32 WMO), WC blocks of 32 input
// channels (CT = 32 WC) and WK segments of every pixel row (the segments' sums are added at the end of the block):
//   4 x 1 x 1  more than 64 output channels;   2 x 2 x 1  up to 64, input channels a multiple of 64;
//   2 x 1 x 2  up to 64 output channels, input channels a multiple of 32;
//   1 x 2 x 2  up to 32 output channels, input channels a multiple of 64;   1 x 1 x 4  up to 32, a multiple of 32.
// Every wave then runs 9 accumulator blocks of 32(oc) x 32(c), one per filter tap: the MFMA A operand of lane l
// is Gs[oc = l%32][pixel + l/32], the B operand of tap (ky,kx) is Xs[c = l%32][that pixel shifted by (ky,kx)].
// The odd pitches put the 32 lanes of a half-wave on 32 different LDS banks for both reads.  The patch is loaded
// once and serves all nine taps, so no im2col gather or bounds test is left in the MFMA loop.
// The pixel range is split over blockIdx.z into partial sums kept tap-major ([oc][tap][c], coalesced stores);
// a second kernel adds the partials in split order and writes dw in its [oc][c][tap] order.
//
// Staging: thread t owns float4 column t % 16 of rows t/16 + 16u of either operand, so every address is a
// per-thread constant plus a wave-uniform step.  The next stage's global loads are issued before the MFMA loop of
// the current stage and held in registers until that loop is done.  That fixes the shapes served here (stages of at
// most 64 pixels over 3 or 4 patch rows: rows of at most 64 floats, or segments of wider rows, see SEG below); the
// implicit-GEMM kernel takes the rest.
#pragma once
#include "igemm_core.hpp"

namespace wgp {
using igemm::FastDiv;
using igemm::f32x16;

constexpr int KH = 3, KW = 3, KK = 9;
constexpr int NT = 256;                     // threads per block
constexpr int LPR = 16, RPP = NT / LPR;     // lanes per staged row, rows covered by one pass of the block
constexpr int SLACK = 64;                   // floats behind the last plane that the look-ahead read may touch
constexpr size_t LDS_BUDGET = 72 * 1024;    // per block, so that two blocks share a CU

using igemm::ldg4;

struct Params {
    const float* x;
    const float* g;
    float* part;
    int Cin, H, W, Cout, oh, ow, sh, sw, ph, pw;
    int R, PW, PLANE, GP, Kst;  // rows per stage, patch width, plane pitch, g pitch, pixels per stage
    int stages, sps, spi;       // all stages, stages per split, stages per image
    int xcd_chunk;              // blocks / 8 when that divides (see the kernel), else 0
    int XRn;                    // NARROW kernels: patch rows per stage (a whole image)
    int segw, nseg;             // SEG kernels: pixels per row segment, segments per row
    FastDiv div_spi, div_xr, div_nseg;
    i64 part_stride;
};

// XR = patch rows per stage = (R - 1) * sh + 3; WMO x WC x WK = wave layout (see the top of the file).
// NARROW (maps of at most 64 pixels with rows of at most 16 floats, XR unused): a stage is one whole image, and the patch is
// staged by (channel, row) pairs, 4 lanes per row and 64 pairs per pass, instead of 16 lanes per row: with 8-float rows
// the regular map would leave 14 of 16 lanes idle and could hold only 4 of the image's 10 patch rows.
// PAIRS > 0 (unit column stride, a wave's row segment = 2 PAIRS pixels): the pixel loop of a row is unrolled, see compute.
// SEG (rows of more than 64 floats; unit column stride, padding 1, XR = 3): a stage is one SEGMENT of segw pixels of one output
// row.  The patch under it is staged with four columns of halo on either side, taken from the neighbouring segments or zero
// past the ends of the row: thread column q holds image columns sg * segw - 4 + 4q .. + 3, so LDS column j of a patch row is
// image column sg * segw - 4 + j and every column of the patch is rewritten by every stage.
template <int XR, int WMO, int WC, int WK, bool NARROW = false, int PAIRS = 0, bool SEG = false>
__global__ __launch_bounds__(NT, 2) void wgrad_patch_kernel(const Params p) {
    static_assert(WMO * WC * WK == 4, "four waves");
    static_assert(!SEG || (!NARROW && XR == 3), "segment stages: one output row, three patch rows");
    static_assert(!NARROW || WC == 1, "narrow staging holds 32 channel planes");
    constexpr int BM = 32 * WMO, CT = 32 * WC;
    constexpr int NG = BM / RPP, NXC = CT / RPP;
    constexpr int NXN = 5;  // NARROW: passes of 64 (channel, row) pairs; 32 channels x at most 10 rows
    constexpr int NX = NARROW ? NXN : NXC * XR;
    FX_DYNAMIC_SMEM(float, smem);
    float* Gs = smem;
    float* Xs = smem + BM * p.GP;
    const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5, l32 = lane & 31;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // in a scalar register, with everything derived from it
    // Workgroup ids go to the 8 XCDs round-robin; remapped so that each XCD takes a contiguous range of
    // (split, oc tile, channel tile) triples: the channel tiles of one split read the same rows of g through one L2.
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
    const int L = p.oh * p.ow;
    const int k4 = p.Kst >> 2, w4 = SEG ? (p.segw >> 2) + 2 : p.W >> 2;

    for (int i = tid; i < CT * p.PLANE + SLACK; i += NT) Xs[i] = 0.f;  // the padding columns stay zero from here on
    f32x16 acc[KK];
#pragma unroll
    for (int t = 0; t < KK; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[t][e] = 0.f;
    __syncthreads();

    // registers of the stage in flight and the per-thread constants of its addresses
    const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
    float4 gv[NG], xv[NX];
    const int pq = tid & (LPR - 1), prow = tid / LPR;
    const bool g_lane = pq < k4, x_lane = pq < w4;
    const bool full_m = oc0 + BM <= p.Cout;
    const uint32_t g_off = g_lane ? (uint32_t)(prow * L + 4 * pq) * 4u : 0u;
    uint32_t x_off = x_lane ? (uint32_t)(prow * p.H * p.W + 4 * pq) * 4u : 0u;
    uint32_t x_off0 = x_lane ? (uint32_t)(4 * pq) * 4u : 0u;  // the same columns in the first plane of a pass
    bool col_zero = false;  // SEG: this thread's columns of the stage in flight lie past an end of the row
    // ragged input-channel counts come only with the 1 x 1 x 4 layout; elsewhere this folds to a constant and the
    // staging code carries no channel tests (they cost the 128-row layout a fifth of its speed in registers)
    constexpr bool RAGGED_C = WMO == 1 && WC == 1;  // 1 x 1 x 4: the only layout the planner gives ragged counts to
    const bool full_c = !RAGGED_C || c0 + CT <= p.Cin;
    const int g_dst0 = prow * p.GP + 4 * pq;
    const int x_dst0 = BM * p.GP + prow * p.PLANE + (SEG ? 0 : p.pw) + 4 * pq;
    // NARROW: float4 column and first (channel, row) pair of this thread
    const int npq = tid & 3, npp = tid >> 2;
    const bool nx_lane = npq < ((p.W + 3) >> 2);
    const int nxcol = min(4 * npq, p.W - 4), npairs = CT * p.XRn;
    auto prefetch = [&](int s) {
        const int b = (int)p.div_spi.div((uint32_t)s);
        int oy0 = (s - b * p.spi) * p.R, sg = 0;
        if constexpr (SEG) {
            const int rest = s - b * p.spi;
            oy0 = (int)p.div_nseg.div((uint32_t)rest);
            sg = rest - oy0 * p.nseg;
            const int cx = sg * p.segw - 4 + 4 * pq;  // first image column of this thread's four
            col_zero = cx < 0 || cx >= p.W;
            x_off = x_lane && !col_zero ? (uint32_t)(prow * p.H * p.W + cx) * 4u : 0u;
            x_off0 = x_lane && !col_zero ? (uint32_t)cx * 4u : 0u;
        }
        const int iy0 = oy0 * p.sh - p.ph;
        const float* gsrc = p.g + ((i64)b * p.Cout + oc0) * L + (i64)oy0 * p.ow + sg * (SEG ? p.segw : 0);
        const float* xsrc = p.x + ((i64)b * p.Cin + c0) * p.H * p.W;
#pragma unroll
        for (int u = 0; u < NG; ++u) {
            // rows past the last output channel are never loaded: a pass of 16 rows that starts past it reads row oc0
            // instead (block-uniform choice), a thread whose own row is past it reads the first row of its pass
            const bool pass_in = full_m || oc0 + u * RPP < p.Cout;
            const bool ok = full_m || oc0 + prow + u * RPP < p.Cout;
            gv[u] = ldg4(pass_in ? gsrc + (i64)u * RPP * L : gsrc, ok ? g_off : 0u);
        }
        if constexpr (NARROW) {
#pragma unroll
            for (int u = 0; u < NXN; ++u) {
                const int pair = u * 64 + npp;
                const int c = (int)p.div_xr.div((uint32_t)pair), iy = iy0 + pair - c * p.XRn;
                const bool ok = nx_lane && pair < npairs && iy >= 0 && iy < p.H && (full_c || c0 + c < p.Cin);
                xv[u] = ldg4(xsrc, ok ? (uint32_t)((c * p.H + iy) * p.W + nxcol) * 4u : 0u);
            }
        }
#pragma unroll
        for (int r = 0; r < (NARROW ? 0 : XR); ++r) {
            const int iy = iy0 + r;
            const bool row_ok = iy >= 0 && iy < p.H;  // wave-uniform
#pragma unroll
            for (int cu = 0; cu < NXC; ++cu) {
                // planes past the last input channel are never loaded (same rule as for the rows of g above) and never
                // parked: their LDS planes keep the zeros of the initial fill
                const bool pass_in = full_c || c0 + cu * RPP < p.Cin;
                const bool ok = full_c || c0 + prow + cu * RPP < p.Cin;
                if (row_ok) xv[r * NXC + cu] = ldg4(xsrc + ((i64)(pass_in ? cu * RPP : 0) * p.H + iy) * p.W, ok ? x_off : x_off0);
                else xv[r * NXC + cu] = zero4;
            }
        }
    };
    auto park = [&]() {
        int gd = g_dst0, xd = x_dst0;
        FX_PIN_VGPR2(gd, xd);  // recompute the row addresses here instead of keeping 14 of them alive
        if (g_lane) {
#pragma unroll
            for (int u = 0; u < NG; ++u) {
                const bool ok = full_m || oc0 + prow + u * RPP < p.Cout;
                const float4 v = ok ? gv[u] : zero4;
                float* d = smem + gd + u * RPP * p.GP;
                d[0] = v.x; d[1] = v.y; d[2] = v.z; d[3] = v.w;
            }
        }
        if constexpr (NARROW) {
            if (nx_lane) {
#pragma unroll
                for (int u = 0; u < NXN; ++u) {
                    const int pair = u * 64 + npp;
                    const int c = (int)p.div_xr.div((uint32_t)pair), r = pair - c * p.XRn, iy = r - p.ph;
                    if (pair < npairs && (full_c || c0 + c < p.Cin)) {  // rows above and below the image are written as zeros
                        const float4 v = iy >= 0 && iy < p.H ? xv[u] : zero4;
                        float* d = Xs + c * p.PLANE + r * p.PW + p.pw + nxcol;
                        d[0] = v.x; d[1] = v.y; d[2] = v.z; d[3] = v.w;
                    }
                }
            }
        }
        if (!NARROW && x_lane) {
#pragma unroll
            for (int r = 0; r < XR; ++r)
#pragma unroll
                for (int cu = 0; cu < NXC; ++cu) {
                    if (!(full_c || c0 + prow + cu * RPP < p.Cin)) continue;
                    const float4 v = SEG && col_zero ? zero4 : xv[r * NXC + cu];
                    float* d = smem + xd + cu * RPP * p.PLANE + r * p.PW;
                    d[0] = v.x; d[1] = v.y; d[2] = v.z; d[3] = v.w;
                }
        }
    };

    const int wmo = wave % WMO, wc = (wave / WMO) % WC, wk = wave / (WMO * WC);
    const int seg = (SEG ? p.segw : p.ow) / WK;  // pixels of a row that this wave covers (a multiple of 2)
    const float* ga = Gs + (wmo * 32 + l32) * p.GP + half + wk * seg;
    const float* xb = Xs + (wc * 32 + l32) * p.PLANE + (half + wk * seg) * p.sw + (SEG ? 4 - p.pw : 0);
    const int sw2 = 2 * p.sw;
    // One stage of MFMA work.  Two register sets alternate: while the MFMAs of one pixel pair run, the operands of
    // the next pair are read from LDS into the other set.  The reads past the end of a row land in the pitch
    // padding or in the slack behind the planes and are never used.
    auto compute = [&]() {
        if constexpr (PAIRS > 0) {
            // Unit column stride and a row segment of 2 PAIRS pixels, unrolled: every LDS address is a row pointer plus an
            // immediate, and of the three patch columns under a pixel pair the last one is the next pair's first, so a
            // pair costs 7 LDS reads (1 of g, 3 middle, 3 new right columns) for its 9 MFMAs and no address arithmetic.
            for (int r = 0; r < p.R; ++r) {
                const float* gr = ga + r * p.ow;
                const float* xk[KH];
                xk[0] = xb + r * p.sh * p.PW;
                xk[1] = xk[0] + p.PW;
                xk[2] = xk[1] + p.PW;
                float a[PAIRS], mid[PAIRS][KH], col[PAIRS + 1][KH];
                auto rd = [&](int j) __attribute__((always_inline)) {
                    a[j] = gr[2 * j];
#pragma unroll
                    for (int ky = 0; ky < KH; ++ky) {
                        mid[j][ky] = xk[ky][2 * j + 1];
                        col[j + 1][ky] = xk[ky][2 * j + 2];
                    }
                    __builtin_amdgcn_sched_barrier(0);
                };
#pragma unroll
                for (int ky = 0; ky < KH; ++ky) col[0][ky] = xk[ky][0];
                rd(0);
#pragma unroll
                for (int j = 0; j < PAIRS; ++j) {
                    if (j + 1 < PAIRS) rd(j + 1);
#pragma unroll
                    for (int ky = 0; ky < KH; ++ky) {
                        acc[ky * KW + 0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[j], col[j][ky], acc[ky * KW + 0], 0, 0, 0);
                        acc[ky * KW + 1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[j], mid[j][ky], acc[ky * KW + 1], 0, 0, 0);
                        acc[ky * KW + 2] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[j], col[j + 1][ky], acc[ky * KW + 2], 0, 0, 0);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            return;
        }
        for (int r = 0; r < p.R; ++r) {
            const float* gr = ga + r * p.ow;
            const float* x0 = xb + r * p.sh * p.PW;
            const float* x1 = x0 + p.PW;
            const float* x2 = x1 + p.PW;
            float a0, b0[KK], a1, b1[KK];
            auto rd = [&](float& a, float (&b)[KK], int j) {
                a = gr[j];
#pragma unroll
                for (int kx = 0; kx < KW; ++kx) { b[kx] = x0[kx]; b[KW + kx] = x1[kx]; b[2 * KW + kx] = x2[kx]; }
                x0 += sw2; x1 += sw2; x2 += sw2;
                __builtin_amdgcn_sched_barrier(0);
            };
            auto mma = [&](float a, const float (&b)[KK]) {
#pragma unroll
                for (int t = 0; t < KK; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b[t], acc[t], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            };
            rd(a0, b0, 0);
            int j = 0;
            for (; j + 4 <= seg; j += 4) {
                rd(a1, b1, j + 2);
                mma(a0, b0);
                rd(a0, b0, j + 4);
                mma(a1, b1);
            }
            if (j < seg) mma(a0, b0);
        }
    };

    const int s_beg = bzi * p.sps, s_end = min(p.stages, s_beg + p.sps);
    if (s_beg < s_end) {
        prefetch(s_beg);
        park();
    }
    __syncthreads();
    for (int s = s_beg; s < s_end; ++s) {
        const bool more = s + 1 < s_end;
        if (more) prefetch(s + 1);
        // The other block on this CU may be staging: its address arithmetic must not win the issue slot over
        // this wave's MFMAs, so the MFMA loop runs at raised wave priority.
        __builtin_amdgcn_s_setprio(3);
        compute();
        __builtin_amdgcn_s_setprio(0);
        __syncthreads();
        if (more) park();
        __syncthreads();
    }

    // The WK waves that split the pixel rows hold partial sums of the same outputs: added here in order of wk, tap by
    // tap through LDS (the stage buffers are free after the loop's last barrier), so a block leaves one partial sum.
    if constexpr (WK > 1) {
        float* red = smem;  // [4 waves][16][64]
#pragma unroll
        for (int t = 0; t < KK; ++t) {
#pragma unroll
            for (int e = 0; e < 16; ++e) red[(wave * 16 + e) * 64 + lane] = acc[t][e];
            __syncthreads();
            if (wk == 0) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    float v = acc[t][e];
#pragma unroll
                    for (int q = 1; q < WK; ++q) v = v + red[((wave + q * WMO * WC) * 16 + e) * 64 + lane];
                    acc[t][e] = v;
                }
            }
            __syncthreads();
        }
        if (wk != 0) return;
    }
    float* out = p.part + (i64)bzi * p.part_stride;
    const int ldo = KK * p.Cin;
#pragma unroll
    for (int t = 0; t < KK; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const int oc = oc0 + wmo * 32 + igemm::Mfma<float>::row(e, lane);
            if (oc < p.Cout && (!RAGGED_C || c0 + wc * 32 + l32 < p.Cin)) out[(i64)oc * ldo + t * p.Cin + c0 + wc * 32 + l32] = acc[t][e];
        }
}

// A second, short result behind every partial (the bias sums of the masked kernels: nb floats at offset n of each split,
// splits `stride` floats apart; stride 0 = the partials are n apart and there is no tail).  The blocks past the main ones
// of a reduce launch add it over the splits, G threads per output like the main sum.
struct ReduceTail {
    i64 stride = 0;
    float* db = nullptr;
    int nb = 0;
};
inline i64 tail_blocks(const ReduceTail& t, int outputs_per_block) { return t.db ? fx::ceil_div((i64)t.nb, (i64)outputs_per_block) : 0; }
template <int G>
__device__ __forceinline__ void reduce_tail(const float* __restrict__ part, int n, int splits, const ReduceTail& t, int block) {
    constexpr int COLS = 256 / G;
    __shared__ float smt[G][COLS];
    const int col = threadIdx.x % COLS, g = threadIdx.x / COLS;
    const int i = block * COLS + col;
    float s = 0.f;
    if (i < t.nb) {
        int z = g;
        for (; z + 7 * G < splits; z += 8 * G) {  // eight loads in flight, added in order
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = part[(i64)(z + u * G) * t.stride + n + i];
#pragma unroll
            for (int u = 0; u < 8; ++u) s = s + v[u];
        }
        for (; z < splits; z += G) s = s + part[(i64)z * t.stride + n + i];
    }
    smt[g][col] = s;
    __syncthreads();
    if (g == 0 && i < t.nb) {
        float v = smt[0][col];
#pragma unroll
        for (int u = 1; u < G; ++u) v = v + smt[u][col];
        t.db[i] = v;
    }
}

// out[(oc*Cin + c)*KK + t] = sum_z part[z][oc][t][c], splits added in order.
__global__ __launch_bounds__(256) void wgrad_patch_reduce_kernel(const float* __restrict__ part, float* __restrict__ out, int n,
                                                                 int splits, int Cin, FastDiv div_row, FastDiv div_cin,
                                                                 const ReduceTail tail = ReduceTail()) {
    const int main_blocks = (n + 255) / 256;
    if ((int)blockIdx.x >= main_blocks) { reduce_tail<1>(part, n, splits, tail, blockIdx.x - main_blocks); return; }
    const i64 ps = tail.stride ? tail.stride : n;
    const int j = blockIdx.x * 256 + threadIdx.x;
    if (j >= n) return;
    float s = 0.f;
    int z = 0;
    for (; z + 8 <= splits; z += 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = part[(i64)(z + u) * ps + j];
#pragma unroll
        for (int u = 0; u < 8; ++u) s = s + v[u];
    }
    for (; z < splits; ++z) s = s + part[(i64)z * ps + j];
    const int oc = (int)div_row.div((uint32_t)j), rem = j - oc * (KK * Cin);
    const int t = (int)div_cin.div((uint32_t)rem), c = rem - t * Cin;
    out[((i64)oc * Cin + c) * KK + t] = s;
}

// The same sum for few outputs and many partials: G threads share one output, thread g adds partials g, g+G, ... in
// order, then the G sums are added in order of g (fixed grouping: reproducible run to run).
template <int G>
__global__ __launch_bounds__(256) void wgrad_patch_reduce_grouped_kernel(const float* __restrict__ part, float* __restrict__ out, int n,
                                                                         int splits, int Cin, FastDiv div_row, FastDiv div_cin,
                                                                         const ReduceTail tail = ReduceTail()) {
    constexpr int COLS = 256 / G;
    const int main_blocks = (n + COLS - 1) / COLS;
    if ((int)blockIdx.x >= main_blocks) { reduce_tail<G>(part, n, splits, tail, blockIdx.x - main_blocks); return; }
    const i64 ps = tail.stride ? tail.stride : n;
    __shared__ float sm[G][COLS];
    const int col = threadIdx.x % COLS, g = threadIdx.x / COLS;
    const int j = blockIdx.x * COLS + col;
    float s = 0.f;
    if (j < n) {
        int z = g;
        for (; z + 7 * G < splits; z += 8 * G) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = part[(i64)(z + u * G) * ps + j];
#pragma unroll
            for (int u = 0; u < 8; ++u) s = s + v[u];
        }
        for (; z < splits; z += G) s = s + part[(i64)z * ps + j];
    }
    sm[g][col] = s;
    __syncthreads();
    if (g == 0 && j < n) {
        float t = sm[0][col];
#pragma unroll
        for (int u = 1; u < G; ++u) t = t + sm[u][col];
        const int oc = (int)div_row.div((uint32_t)j), rem = j - oc * (KK * Cin);
        const int tap = (int)div_cin.div((uint32_t)rem), c = rem - tap * Cin;
        out[((i64)oc * Cin + c) * KK + tap] = t;
    }
}

// The grouped sum over four adjacent outputs per thread (n and Cin multiples of 4, so the four share their output channel and
// tap): 16-byte loads, a group's 16 threads cover 256 contiguous bytes of a partial.  Same grouping and order as above.
template <int G>
__global__ __launch_bounds__(256) void wgrad_patch_reduce_vec_kernel(const float* __restrict__ part, float* __restrict__ out, int n,
                                                                     int splits, int Cin, FastDiv div_row, FastDiv div_cin,
                                                                     const ReduceTail tail = ReduceTail()) {
    constexpr int COLS = 256 / G;
    const int main_blocks = (n + 4 * COLS - 1) / (4 * COLS);
    if ((int)blockIdx.x >= main_blocks) { reduce_tail<G>(part, n, splits, tail, blockIdx.x - main_blocks); return; }
    const i64 ps = tail.stride ? tail.stride : n;
    __shared__ float4 sm[G][COLS];
    const int col = threadIdx.x % COLS, g = threadIdx.x / COLS;
    const int j = (blockIdx.x * COLS + col) * 4;
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
    if (j < n) {
        int z = g;
        for (; z + 7 * G < splits; z += 8 * G) {
            float4 v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = *reinterpret_cast<const float4*>(part + (i64)(z + u * G) * ps + j);
#pragma unroll
            for (int u = 0; u < 8; ++u) { s.x = s.x + v[u].x; s.y = s.y + v[u].y; s.z = s.z + v[u].z; s.w = s.w + v[u].w; }
        }
        for (; z < splits; z += G) {
            const float4 v = *reinterpret_cast<const float4*>(part + (i64)z * ps + j);
            s.x = s.x + v.x; s.y = s.y + v.y; s.z = s.z + v.z; s.w = s.w + v.w;
        }
    }
    sm[g][col] = s;
    __syncthreads();
    if (g == 0 && j < n) {
        float4 t = sm[0][col];
#pragma unroll
        for (int u = 1; u < G; ++u) { const float4 v = sm[u][col]; t.x = t.x + v.x; t.y = t.y + v.y; t.z = t.z + v.z; t.w = t.w + v.w; }
        const int oc = (int)div_row.div((uint32_t)j), rem = j - oc * (KK * Cin);
        const int tap = (int)div_cin.div((uint32_t)rem), c = rem - tap * Cin;
        float* o = out + ((i64)oc * Cin + c) * KK + tap;
        o[0] = t.x; o[KK] = t.y; o[2 * KK] = t.z; o[3 * KK] = t.w;
    }
}

struct Plan {
    bool ok = false;
    int R = 1, PR = 0, PW = 0, PLANE = 0, GP = 0, Kst = 0, splits = 1, sps = 1, stages = 0;
    int WMO = 4, WC = 1, WK = 1;  // wave layout
    bool narrow = false;          // whole-image stages with the (channel, row) pair staging
    int segw = 0, nseg = 0;       // rows of more than 64 floats: pixels per row segment, segments per row (SEG kernels)
    size_t smem = 0;
    int bm() const { return 32 * WMO; }
    int ct() const { return 32 * WC; }
    int partials() const { return splits; }
};

inline int odd_pitch(int n) { return (n + 30) / 32 * 32 + 1; }  // smallest pitch >= n with pitch % 32 == 1

inline Plan make_plan(int num_cus, i64 B, i64 Cin, i64 H, i64 W, i64 Cout, i64 kh, i64 kw, i64 sh, i64 sw, i64 ph, i64 pw, i64 oh, i64 ow) {
    Plan pl;
    // Input channels: whole blocks of 32; with up to 32 output channels also ragged counts (at most half of the last
    // block's planes unused).  Measured: [256,16,32,32] -> 32 0.100 -> 0.064 ms against the implicit GEMM, but with more
    // output channels the padded block loses ([256,16,32,32] -> 64 0.098 -> 0.113 ms, [128,48,56,56] -> 128 0.549 -> 0.594 ms).
    const bool ragged_c = Cin % 32 != 0;
    if (ragged_c && (Cout > 32 || fx::ceil_div(Cin, (i64)32) * 32 > 2 * Cin)) return pl;
    if (kh != KH || kw != KW || ow % 2 != 0 || W % 4 != 0 || sh > 8 || sw > 8) return pl;
    // Rows of more than 64 floats are walked in segments: the largest divisor of the row that is a multiple of 4 within 24 .. 56
    // pixels (with its two halo vectors a staged patch row then fits the 16 lanes of a staging row).
    i64 segw = 0;
    if (W > 4 * LPR) {
        if (sw != 1 || pw != 1 || ow != W) return pl;
        for (i64 k = 56; k >= 24 && !segw; k -= 4)
            if (ow % k == 0) segw = k;
        if (!segw) return pl;
    }
    // Wave layouts that fit the channel counts, the preferred one first.  Up to 32 output channels: one block of them, the
    // four waves split the input channels and / or the rows; up to 64: two blocks, the other two waves take more input
    // channels or split the rows.  A layout with 64 input channels per block holds only 3 patch rows (64 channel planes x
    // 4 rows would not fit the register file while in flight), which on narrow maps leaves stages too short: then the
    // next layout is tried.
    int cand[2][3], ncand = 0;
    auto add = [&](int a, int b, int c) { cand[ncand][0] = a; cand[ncand][1] = b; cand[ncand][2] = c; ++ncand; };
    const i64 rowlen = segw ? segw : ow;  // pixels of a row in one stage
    if (Cout <= 32) {
        if (Cin % 64 == 0 && rowlen % 4 == 0) add(1, 2, 2);
        if (rowlen % 8 == 0) add(1, 1, 4);
    } else if (Cout <= 64) {
        if (Cin % 64 == 0) add(2, 2, 1);
        if (rowlen % 4 == 0) add(2, 1, 2);
    } else {
        add(4, 1, 1);
    }
    int best = 0;  // the most rows per stage that keep a stage within 64 pixels, max_pr patch rows and the LDS budget
    for (int k = 0; k < ncand && !best; ++k) {
        pl.WMO = cand[k][0]; pl.WC = cand[k][1]; pl.WK = cand[k][2];
        const i64 max_pr = pl.WC == 2 ? 3 : 4;
        for (int R = 1; R <= (segw ? 1 : oh); ++R) {
            if (oh % R || R * rowlen > 4 * LPR || (R - 1) * sh + kh > max_pr) continue;
            if ((R * rowlen) % 4 == 0) best = R;
        }
        // measured at [256,32,32,32] -> 64, stride 2 (16 pixels per stage): 0.063 ms here against 0.050 ms for the implicit GEMM
        // (and with two output rows over five patch rows per stage: 0.063 against 0.053 ms there, 0.192 against 0.156 ms at
        // [128,64,56,56] -> 128 stride 2: a strided patch stages four input values per output pixel)
        if (best * rowlen < 24) best = 0;
        if (!best) continue;
        pl.R = best;
        pl.PR = (int)((best - 1) * sh + kh);
        pl.PW = (int)(segw ? segw + 8 : W + 2 * pw);
        pl.PLANE = odd_pitch(pl.PR * pl.PW);
        pl.Kst = (int)(best * rowlen);
        pl.GP = odd_pitch(pl.Kst);
        pl.smem = ((size_t)pl.bm() * pl.GP + (size_t)pl.ct() * pl.PLANE + SLACK) * sizeof(float);
        if (pl.WK > 1) pl.smem = std::max<size_t>(pl.smem, 4 * 16 * 64 * sizeof(float));  // the closing sum over the row segments
        if (pl.smem > LDS_BUDGET) best = 0;  // 64 planes of 3 x 66 floats: the next layout holds 32 planes
    }
    if (!best && segw) return pl;
    if (segw) {
        pl.segw = (int)segw;
        pl.nseg = (int)(ow / segw);
    }
    if (!best) {
        // maps of at most 64 pixels with rows of at most 16 floats: one whole image per stage (NARROW kernels)
        const i64 L = oh * ow, XRn = (oh - 1) * sh + kh;
        pl.WC = 1;
        if (Cout > 64) { pl.WMO = 4; pl.WK = 1; }
        else if (Cout > 32 && ow % 4 == 0) { pl.WMO = 2; pl.WK = 2; }
        else if (Cout <= 32 && ow % 8 == 0) { pl.WMO = 1; pl.WK = 4; }
        else return pl;
        if (W > 16 || L > 4 * LPR || L < 24 || L % 4 != 0 || XRn > 10) return pl;
        pl.narrow = true;
        best = (int)oh;
        pl.R = best;
        pl.PR = (int)XRn;
        pl.PW = (int)(W + 2 * pw);
        pl.PLANE = odd_pitch(pl.PR * pl.PW);
        pl.Kst = (int)L;
        pl.GP = odd_pitch(pl.Kst);
        pl.smem = ((size_t)pl.bm() * pl.GP + (size_t)pl.ct() * pl.PLANE + SLACK) * sizeof(float);
        if (pl.WK > 1) pl.smem = std::max<size_t>(pl.smem, 4 * 16 * 64 * sizeof(float));
        if (pl.smem > LDS_BUDGET) return pl;
    }
    const i64 BM = pl.bm(), CT = pl.ct();
    if (B * (oh / best) * std::max(1, pl.nseg) > 0x7fffffff) return pl;
    pl.stages = (int)(B * (oh / best) * std::max(1, pl.nseg));
    const i64 tiles = fx::ceil_div(Cin, CT) * fx::ceil_div(Cout, BM);
    const i64 want = (i64)num_cus * 2;
    // at least four stages per block where there are that many: a block's partial sum (and its closing sum over the row
    // segments) is paid once per block
    const i64 splits = std::max<i64>(1, std::min<i64>(want / tiles, std::max<i64>(1, pl.stages / 4)));
    pl.sps = (int)fx::ceil_div((i64)pl.stages, splits);
    pl.splits = (int)fx::ceil_div((i64)pl.stages, (i64)pl.sps);
    if (pl.splits > 65535 || tiles > 65535 || Cout * Cin * KK > 0x7fffffff) return pl;
    pl.ok = true;
    return pl;
}

inline i64 workspace_bytes(const Plan& pl, i64 Cout, i64 Cin) { return (i64)pl.partials() * Cout * Cin * KK * (i64)sizeof(float); }

// x, g and part must be 16-byte aligned.
inline int run(fx_ctx* c, const Plan& pl, const float* x, const float* g, float* dw, float* part, i64 Cin, i64 H, i64 W, i64 Cout,
               i64 sh, i64 sw, i64 ph, i64 pw, i64 oh, i64 ow) {
    Params p;
    p.x = x; p.g = g; p.part = part;
    p.Cin = (int)Cin; p.H = (int)H; p.W = (int)W; p.Cout = (int)Cout; p.oh = (int)oh; p.ow = (int)ow;
    p.sh = (int)sh; p.sw = (int)sw; p.ph = (int)ph; p.pw = (int)pw;
    p.R = pl.R; p.PW = pl.PW; p.PLANE = pl.PLANE; p.GP = pl.GP; p.Kst = pl.Kst;
    p.stages = pl.stages; p.sps = pl.sps; p.spi = (int)(oh / pl.R) * std::max(1, pl.nseg);
    p.segw = pl.segw; p.nseg = std::max(1, pl.nseg);
    p.div_nseg = FastDiv((uint32_t)p.nseg);
    p.div_spi = FastDiv((uint32_t)p.spi);
    p.XRn = pl.PR;
    p.div_xr = FastDiv((uint32_t)pl.PR);
    p.part_stride = Cout * Cin * KK;
    const dim3 grid((unsigned)fx::ceil_div(Cin, (i64)pl.ct()), (unsigned)fx::ceil_div(Cout, (i64)pl.bm()), (unsigned)pl.splits);
    const i64 blocks = (i64)grid.x * grid.y * grid.z;
    p.xcd_chunk = blocks % 8 == 0 && blocks <= 0x7fffffff ? (int)(blocks / 8) : 0;
#define FX_WGP_LAUNCH(XRV, A, B_, C_)                                                                                 \
    do {                                                                                                              \
        static const hipError_t attr = hipFuncSetAttribute((const void*)wgrad_patch_kernel<XRV, A, B_, C_>,           \
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_BUDGET); \
        FX_HIP_CHECK(attr);                                                                                           \
        FX_LAUNCH(grid, dim3(NT), pl.smem, c->stream, (p), wgrad_patch_kernel<XRV, A, B_, C_>);                                \
    } while (0)
    const int layout = pl.WMO * 100 + pl.WC * 10 + pl.WK;
    // pixel pairs of a wave's row segment when the unrolled pixel loop applies (unit column stride), else 0
    const i64 rowlen = pl.segw ? pl.segw : ow;
    const int pairs = sw == 1 && !pl.narrow && (rowlen / pl.WK) % 2 == 0 ? (int)(rowlen / pl.WK / 2) : 0;
#define FX_WGP_LAUNCH_PAIRS(XRV, A, B_, C_, PV)                                                                       \
    do {                                                                                                              \
        static const hipError_t attr = hipFuncSetAttribute((const void*)wgrad_patch_kernel<XRV, A, B_, C_, false, PV>, \
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_BUDGET); \
        FX_HIP_CHECK(attr);                                                                                           \
        FX_LAUNCH(grid, dim3(NT), pl.smem, c->stream, (p), wgrad_patch_kernel<XRV, A, B_, C_, false, PV>);                     \
    } while (0)
#define FX_WGP_LAUNCH_NARROW(A, C_)                                                                                   \
    do {                                                                                                              \
        static const hipError_t attr = hipFuncSetAttribute((const void*)wgrad_patch_kernel<0, A, 1, C_, true>,        \
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_BUDGET); \
        FX_HIP_CHECK(attr);                                                                                           \
        FX_LAUNCH(grid, dim3(NT), pl.smem, c->stream, (p), wgrad_patch_kernel<0, A, 1, C_, true>);                             \
    } while (0)
#define FX_WGP_LAUNCH_SEG(A, B_, C_, PV)                                                                              \
    do {                                                                                                              \
        static const hipError_t attr = hipFuncSetAttribute((const void*)wgrad_patch_kernel<3, A, B_, C_, false, PV, true>, \
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_BUDGET); \
        FX_HIP_CHECK(attr);                                                                                           \
        FX_LAUNCH(grid, dim3(NT), pl.smem, c->stream, (p), wgrad_patch_kernel<3, A, B_, C_, false, PV, true>);        \
    } while (0)
    if (pl.segw) {
        FX_REQUIRE(pl.PR == 3, "wgrad patch kernel: segment stages hold three patch rows");
        if (layout == 411 && pairs == 28) FX_WGP_LAUNCH_SEG(4, 1, 1, 28);
        else if (layout == 411 && pairs == 16) FX_WGP_LAUNCH_SEG(4, 1, 1, 16);
        else if (layout == 411) FX_WGP_LAUNCH_SEG(4, 1, 1, 0);
        else if (layout == 221 && pairs == 28) FX_WGP_LAUNCH_SEG(2, 2, 1, 28);
        else if (layout == 221 && pairs == 16) FX_WGP_LAUNCH_SEG(2, 2, 1, 16);
        else if (layout == 221) FX_WGP_LAUNCH_SEG(2, 2, 1, 0);
        else if (layout == 212) FX_WGP_LAUNCH_SEG(2, 1, 2, 0);
        else if (layout == 122) FX_WGP_LAUNCH_SEG(1, 2, 2, 0);
        else if (layout == 114) FX_WGP_LAUNCH_SEG(1, 1, 4, 0);
        else FX_REQUIRE(false, "wgrad patch kernel: unexpected wave layout %d", layout);
    } else if (pl.narrow && layout == 411) FX_WGP_LAUNCH_NARROW(4, 1);
    else if (pl.narrow && layout == 212) FX_WGP_LAUNCH_NARROW(2, 2);
    else if (pl.narrow && layout == 114) FX_WGP_LAUNCH_NARROW(1, 4);
    else if (pl.narrow) FX_REQUIRE(false, "wgrad patch kernel: unexpected narrow layout %d", layout);
    else if (layout == 411 && pl.PR == 3 && pairs == 28) FX_WGP_LAUNCH_PAIRS(3, 4, 1, 1, 28);
    else if (layout == 411 && pl.PR == 4 && pairs == 14) FX_WGP_LAUNCH_PAIRS(4, 4, 1, 1, 14);
    else if (layout == 221 && pl.PR == 3 && pairs == 28) FX_WGP_LAUNCH_PAIRS(3, 2, 2, 1, 28);
    else if (layout == 411 && pl.PR == 3) FX_WGP_LAUNCH(3, 4, 1, 1);
    else if (layout == 411) FX_WGP_LAUNCH(4, 4, 1, 1);
    else if (layout == 221 && pl.PR == 3) FX_WGP_LAUNCH(3, 2, 2, 1);
    else if (layout == 212 && pl.PR == 3) FX_WGP_LAUNCH(3, 2, 1, 2);
    else if (layout == 212) FX_WGP_LAUNCH(4, 2, 1, 2);
    else if (layout == 122) FX_WGP_LAUNCH(3, 1, 2, 2);
    else if (layout == 114 && pl.PR == 3) FX_WGP_LAUNCH(3, 1, 1, 4);
    else if (layout == 114) FX_WGP_LAUNCH(4, 1, 1, 4);
    else FX_REQUIRE(false, "wgrad patch kernel: unexpected wave layout %d", layout);
#undef FX_WGP_LAUNCH
#undef FX_WGP_LAUNCH_PAIRS
#undef FX_WGP_LAUNCH_NARROW
#undef FX_WGP_LAUNCH_SEG
    FX_LAUNCH_CHECK();
    const int n = (int)p.part_stride;
    const FastDiv div_row((uint32_t)(KK * Cin)), div_cin((uint32_t)Cin);
    // the two 4-byte kernels serve partial sums that are not 16-byte addressable; between them, measured: with 256 partials of
    // 73 728 outputs the single chain per output is the faster one (0.095 vs 0.106 ms for the whole pass at [64,128,28,28] -> 64),
    // with 1024 partials of 18 432 outputs the grouped sum wins (0.118 vs 0.141 ms)
    // measured: the 16-byte grouped sum beats both kernels below wherever it applies (0.4845 -> 0.4786 ms for the whole pass at
    // [128,64,56,56] -> 128 with 256 partials, 0.1996 -> 0.188 ms at [256,64,32,32] -> 64)
    if (n % 4 == 0 && Cin % 4 == 0 && fx::aligned16(part)) {
        FX_LAUNCH(dim3((unsigned)fx::ceil_div((i64)n, 64)), dim3(256), 0, c->stream, (part, dw, n, pl.partials(), (int)Cin, div_row, div_cin), wgrad_patch_reduce_vec_kernel<16>);
    } else if (pl.partials() >= 512 && n <= (1 << 17))
        FX_LAUNCH(dim3((unsigned)fx::ceil_div((i64)n, 16)), dim3(256), 0, c->stream, (part, dw, n, pl.partials(), (int)Cin, div_row, div_cin), wgrad_patch_reduce_grouped_kernel<16>);
    else
        FX_LAUNCH(dim3((unsigned)fx::ceil_div((i64)n, 256)), dim3(256), 0, c->stream, (part, dw, n, pl.partials(), (int)Cin, div_row, div_cin), wgrad_patch_reduce_kernel);
    FX_LAUNCH_CHECK();
    return FX_OK;
}

}  // namespace wgp
