// Weight gradient of a 3x3 convolution (f64) on v_mfma_f64_16x16x4_f64 with both operands staged in LDS in their natural
// layouts; the f64 twin of wgp::wgrad_patch_kernel (wgrad_patch.hpp), same product
//   dw[oc][c][ky][kx] = sum over (b, oy, ox) of g[b][oc][oy][ox] * x[b][c][oy*sh+ky-ph][ox+kx-pw]
// (grad_out_2d . im2col(x)^T in the reference, src/backend/storage/extensions/convolutions.rs:296-338).
//
// The f64 MFMA adds a 16(oc) x 4(pixel) by 4(pixel) x 16(c) product to a 16 x 16 block: lane l holds g[oc = l%16][pixel + l/16]
// and x[c = l%16][that pixel shifted by the tap], one double each, and 4 of the 256 sums (oc = 4e + l/16, c = l%16).
// One stage = one output row of one image (unit column stride, row length a multiple of 8 between 24 and 64).  A block
// (4 waves) copies, per stage,
//   Gs[oc][pixel]      64 output-channel rows of g                      (pitch GP odd)
//   Xs[c][row][col]    16 input-channel planes of the 3 zero-padded input rows those pixels touch (pitch PLANE odd)
// and its waves are laid out 2 x 2: two blocks of 32 output channels x the two halves of the pixel row (the halves' sums
// are added in a fixed order when the block ends).  Every wave keeps 2 x 9 accumulator blocks (32 oc x 16 c, one per tap:
// 144 registers) and runs, per group of 4 pixels, 18 MFMAs on 2 + 9 LDS reads.  The pixel loop is unrolled: every LDS
// address is a row pointer plus an immediate.  The pixel range is split over blockIdx.z into partial sums kept tap-major; a
// second kernel adds them in split order and writes dw in its [oc][c][tap] order.
#pragma once
#include <cstdlib>

#include "igemm_core.hpp"

namespace wgd {
using igemm::FastDiv;
using igemm::f64x4;

constexpr int KK = 9, NT = 256, BM = 64, CT = 16;
constexpr int SLACK = 16;
constexpr size_t LDS_BUDGET = 72 * 1024;

struct Params {
    const double* x;
    const double* g;
    double* part;
    int Cin, H, W, Cout, oh, ow, sh, ph, pw;
    int PW, PLANE, GP;
    int stages, sps;    // all stages (B * oh), stages per split
    int xcd_chunk;      // blocks / 8 when that divides, else 0
    FastDiv div_oh;
    i64 part_stride;
};

__device__ __forceinline__ double2 ldg2(const double* base, uint32_t byteoff) {
    typedef __attribute__((address_space(1))) const char gchar;
    typedef double v2 __attribute__((ext_vector_type(2)));
    typedef __attribute__((address_space(1))) const v2 gv2;
    const v2 v = *(gv2*)((gchar*)base + byteoff);
    return make_double2(v.x, v.y);
}

// NK = groups of 4 pixels in a wave's half row (ow = 8 NK)
template <int NK>
__global__ __launch_bounds__(NT, 2) void wgrad_patch_f64_kernel(const Params p) {
    constexpr int NG = BM / 8, NXC = CT / 8, XR = 3;
    FX_DYNAMIC_SMEM(double, smem);
    double* Gs = smem;
    double* Xs = smem + BM * p.GP;
    const int tid = threadIdx.x, lane = tid & 63, kq = lane >> 4, l16 = lane & 15;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wmo = wave & 1, wk = wave >> 1;
    // Workgroup ids go to the 8 XCDs round-robin; remapped so that each XCD takes a contiguous range of (split, oc tile,
    // channel tile) triples: the channel tiles of one split read the same rows of g through one L2.
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

    for (int i = tid; i < CT * p.PLANE + SLACK; i += NT) Xs[i] = 0.;  // the padding columns stay zero from here on
    f64x4 acc[2][KK];
#pragma unroll
    for (int o = 0; o < 2; ++o)
#pragma unroll
        for (int t = 0; t < KK; ++t)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[o][t][e] = 0.;
    __syncthreads();

    // staging: thread t owns the pair of doubles t % 32 of rows t / 32 + 8u of either operand
    const double2 zero2 = make_double2(0., 0.);
    double2 gv[NG], xv[NXC * XR];
    const int pq = tid & 31, prow = tid >> 5;
    const bool g_lane = pq < (p.ow >> 1), x_lane = pq < (p.W >> 1);
    const uint32_t g_off = g_lane ? (uint32_t)(prow * L + 2 * pq) * 8u : 0u;
    const uint32_t x_off = x_lane ? (uint32_t)(prow * p.H * p.W + 2 * pq) * 8u : 0u;
    const int g_dst0 = prow * p.GP + 2 * pq;
    const int x_dst0 = BM * p.GP + prow * p.PLANE + p.pw + 2 * pq;
    auto prefetch = [&](int s) __attribute__((always_inline)) {
        const int b = (int)p.div_oh.div((uint32_t)s);
        const int oy = s - b * p.oh;
        const int iy0 = oy * p.sh - p.ph;
        const double* gsrc = p.g + ((i64)b * p.Cout + oc0) * L + (i64)oy * p.ow;
        const double* xsrc = p.x + ((i64)b * p.Cin + c0) * p.H * p.W;
#pragma unroll
        for (int u = 0; u < NG; ++u) gv[u] = ldg2(gsrc + (i64)u * 8 * L, g_off);
#pragma unroll
        for (int r = 0; r < XR; ++r) {
            const int iy = iy0 + r;
            const bool row_ok = iy >= 0 && iy < p.H;  // scalar
#pragma unroll
            for (int cu = 0; cu < NXC; ++cu) {
                if (row_ok) xv[r * NXC + cu] = ldg2(xsrc + ((i64)cu * 8 * p.H + iy) * p.W, x_off);
                else xv[r * NXC + cu] = zero2;
            }
        }
    };
    auto park = [&]() __attribute__((always_inline)) {
        int gd = g_dst0, xd = x_dst0;
        FX_PIN_VGPR2(gd, xd);  // recompute the row addresses here instead of keeping them alive
        if (g_lane) {
#pragma unroll
            for (int u = 0; u < NG; ++u) {
                double* d = smem + gd + u * 8 * p.GP;
                d[0] = gv[u].x;
                d[1] = gv[u].y;
            }
        }
        if (x_lane) {
#pragma unroll
            for (int r = 0; r < XR; ++r)
#pragma unroll
                for (int cu = 0; cu < NXC; ++cu) {
                    double* d = smem + xd + cu * 8 * p.PLANE + r * p.PW;
                    d[0] = xv[r * NXC + cu].x;
                    d[1] = xv[r * NXC + cu].y;
                }
        }
    };

    // this wave's half row starts at pixel wk * 4 NK; lane l reads pixel + l / 16 of row (channel) l % 16
    const double* ga0 = Gs + (wmo * 32 + l16) * p.GP + wk * 4 * NK + kq;
    const double* ga1 = ga0 + 16 * p.GP;
    const double* xb0 = Xs + l16 * p.PLANE + wk * 4 * NK + kq;
    // One stage: NK groups of 4 pixels x 3 filter rows.  The operands of a (group, filter row) step -- three patch columns, and
    // with the first filter row the two g values of the group -- are read while the 6 MFMAs of the step before run.
    auto compute = [&]() __attribute__((always_inline)) {
        const double* xk[3] = {xb0, xb0 + p.PW, xb0 + 2 * p.PW};
        double a[NK][2], bv[NK * 3][3];
        auto rd = [&](int st) __attribute__((always_inline)) {  // operands of step st = 3 * group + filter row
            const int j = st / 3, ky = st % 3;
            if (ky == 0) {
                a[j][0] = ga0[4 * j];
                a[j][1] = ga1[4 * j];
            }
#pragma unroll
            for (int kx = 0; kx < 3; ++kx) bv[st][kx] = xk[ky][4 * j + kx];
            __builtin_amdgcn_sched_barrier(0);
        };
        rd(0);
#pragma unroll
        for (int st = 0; st < NK * 3; ++st) {
            if (st + 1 < NK * 3) rd(st + 1);
            const int j = st / 3, ky = st % 3;
#pragma unroll
            for (int o = 0; o < 2; ++o)
#pragma unroll
                for (int kx = 0; kx < 3; ++kx)
                    acc[o][ky * 3 + kx] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[j][o], bv[st][kx], acc[o][ky * 3 + kx], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
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
        compute();
        __syncthreads();
        if (more) park();
        __syncthreads();
    }

    // The two waves that split the pixel row hold partial sums of the same outputs: added here, first half + second half, block
    // by block through LDS (the stage buffers are free after the loop's last barrier), so a block leaves one partial sum.
    {
        double* red = smem;  // [2 waves][4][64]
#pragma unroll
        for (int o = 0; o < 2; ++o)
#pragma unroll
            for (int t = 0; t < KK; ++t) {
                if (wk == 1) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) red[(wmo * 4 + e) * 64 + lane] = acc[o][t][e];
                }
                __syncthreads();
                if (wk == 0) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[o][t][e] = acc[o][t][e] + red[(wmo * 4 + e) * 64 + lane];
                }
                __syncthreads();
            }
        if (wk != 0) return;
    }
    double* out = p.part + (i64)bzi * p.part_stride;
    const int ldo = KK * p.Cin;
#pragma unroll
    for (int o = 0; o < 2; ++o)
#pragma unroll
        for (int t = 0; t < KK; ++t)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int oc = oc0 + wmo * 32 + o * 16 + 4 * e + kq;
                out[(i64)oc * ldo + t * p.Cin + c0 + l16] = acc[o][t][e];
            }
}

// A second, short result behind every partial (the bias sums of the masked kernels: nb doubles at offset n of each split,
// splits `stride` doubles apart; stride 0 = the partials are n apart and there is no tail).  The blocks past the main ones
// of a reduce launch add it over the splits, G threads per output like the main sum.
struct ReduceTail {
    i64 stride = 0;
    double* db = nullptr;
    int nb = 0;
};
inline i64 tail_blocks(const ReduceTail& t, int outputs_per_block) { return t.db ? fx::ceil_div((i64)t.nb, (i64)outputs_per_block) : 0; }
template <int G>
__device__ __forceinline__ void reduce_tail(const double* __restrict__ part, int n, int splits, const ReduceTail& t, int block) {
    constexpr int COLS = 256 / G;
    __shared__ double smt[G][COLS];
    const int col = threadIdx.x % COLS, g = threadIdx.x / COLS;
    const int i = block * COLS + col;
    double s = 0.;
    if (i < t.nb) {
        int z = g;
        for (; z + 7 * G < splits; z += 8 * G) {  // eight loads in flight, added in order
            double v[8];
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
        double v = smt[0][col];
#pragma unroll
        for (int u = 1; u < G; ++u) v = v + smt[u][col];
        t.db[i] = v;
    }
}

// out[(oc*Cin + c)*KK + t] = sum_z part[z][oc][t][c], splits added in order.
__global__ __launch_bounds__(256) void wgrad_f64_reduce_kernel(const double* __restrict__ part, double* __restrict__ out, int n, int splits,
                                                               int Cin, FastDiv div_row, FastDiv div_cin, const ReduceTail tail = ReduceTail()) {
    const int main_blocks = (n + 255) / 256;
    if ((int)blockIdx.x >= main_blocks) { reduce_tail<1>(part, n, splits, tail, blockIdx.x - main_blocks); return; }
    const i64 ps = tail.stride ? tail.stride : n;
    const int j = blockIdx.x * 256 + threadIdx.x;
    if (j >= n) return;
    double s = 0.;
    int z = 0;
    for (; z + 8 <= splits; z += 8) {
        double v[8];
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

// The same sum for many partials of a small output (n and Cin even): the splits are dealt to G groups of threads (group g adds
// splits g, g + G, ... in order), the groups' sums are added in group order through LDS; two adjacent outputs per thread, so a
// group's 16 threads read 256 contiguous bytes of a partial with 16-byte loads.
template <int G>
__global__ __launch_bounds__(256) void wgrad_f64_reduce_vec_kernel(const double* __restrict__ part, double* __restrict__ out, int n, int splits,
                                                                   int Cin, FastDiv div_row, FastDiv div_cin, const ReduceTail tail = ReduceTail()) {
    constexpr int COLS = 256 / G;
    const int main_blocks = (n + 2 * COLS - 1) / (2 * COLS);
    if ((int)blockIdx.x >= main_blocks) { reduce_tail<G>(part, n, splits, tail, blockIdx.x - main_blocks); return; }
    const i64 ps = tail.stride ? tail.stride : n;
    __shared__ double2 sm[G][COLS];
    const int col = threadIdx.x % COLS, g = threadIdx.x / COLS;
    const int j = (blockIdx.x * COLS + col) * 2;
    double2 s = make_double2(0., 0.);
    if (j < n) {
        int z = g;
        for (; z + 7 * G < splits; z += 8 * G) {
            double2 v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = *reinterpret_cast<const double2*>(part + (i64)(z + u * G) * ps + j);
#pragma unroll
            for (int u = 0; u < 8; ++u) { s.x = s.x + v[u].x; s.y = s.y + v[u].y; }
        }
        for (; z < splits; z += G) {
            const double2 v = *reinterpret_cast<const double2*>(part + (i64)z * ps + j);
            s.x = s.x + v.x; s.y = s.y + v.y;
        }
    }
    sm[g][col] = s;
    __syncthreads();
    if (g == 0 && j < n) {
        double2 t = sm[0][col];
#pragma unroll
        for (int u = 1; u < G; ++u) { const double2 v = sm[u][col]; t.x = t.x + v.x; t.y = t.y + v.y; }
        const int oc = (int)div_row.div((uint32_t)j), rem = j - oc * (KK * Cin);
        const int tap = (int)div_cin.div((uint32_t)rem), c = rem - tap * Cin;
        double* o = out + ((i64)oc * Cin + c) * KK + tap;
        o[0] = t.x; o[KK] = t.y;
    }
}

struct Plan {
    bool ok = false;
    int PW = 0, PLANE = 0, GP = 0, NK = 0, splits = 1, sps = 1, stages = 0;
    size_t smem = 0;
};

inline int odd(int n) { return n | 1; }

inline Plan make_plan(int num_cus, i64 B, i64 Cin, i64 H, i64 W, i64 Cout, i64 kh, i64 kw, i64 sh, i64 sw, i64 ph, i64 pw, i64 oh, i64 ow) {
    Plan pl;
    if (kh != 3 || kw != 3 || sw != 1 || sh > 8 || Cin % CT != 0 || Cout % BM != 0 || W % 2 != 0 || W > 64 || ow % 8 != 0 || ow < 24 ||
        ow > 64 || Cout * Cin * KK > 0x7fffffff || B * oh > 0x7fffffff)
        return pl;
    pl.NK = (int)(ow / 8);
    if (pl.NK != 3 && pl.NK != 4 && pl.NK != 7 && pl.NK != 8) return pl;  // instantiated row lengths: 24, 32, 56, 64
    pl.PW = (int)(W + 2 * pw);
    pl.PLANE = odd(3 * pl.PW);
    pl.GP = odd((int)ow);
    pl.smem = ((size_t)BM * pl.GP + (size_t)CT * pl.PLANE + SLACK) * sizeof(double);
    pl.smem = std::max<size_t>(pl.smem, 2 * 4 * 64 * sizeof(double));
    if (pl.smem > LDS_BUDGET) return pl;
    pl.stages = (int)(B * oh);
    const i64 tiles = (Cin / CT) * (Cout / BM);
    const i64 splits = std::max<i64>(1, std::min<i64>((i64)num_cus * 2 / tiles, std::max<i64>(1, pl.stages / 4)));
    pl.sps = (int)fx::ceil_div((i64)pl.stages, splits);
    pl.splits = (int)fx::ceil_div((i64)pl.stages, (i64)pl.sps);
    if (pl.splits > 65535 || Cout / BM > 65535) return pl;
    pl.ok = true;
    return pl;
}

inline i64 workspace_bytes(const Plan& pl, i64 Cout, i64 Cin) { return (i64)pl.splits * Cout * Cin * KK * (i64)sizeof(double); }

// x, g and part must be 16-byte aligned.
inline int run(fx_ctx* c, const Plan& pl, const double* x, const double* g, double* dw, double* part, i64 Cin, i64 H, i64 W, i64 Cout, i64 sh,
               i64 ph, i64 pw, i64 oh, i64 ow) {
    Params p;
    p.x = x; p.g = g; p.part = part;
    p.Cin = (int)Cin; p.H = (int)H; p.W = (int)W; p.Cout = (int)Cout; p.oh = (int)oh; p.ow = (int)ow;
    p.sh = (int)sh; p.ph = (int)ph; p.pw = (int)pw;
    p.PW = pl.PW; p.PLANE = pl.PLANE; p.GP = pl.GP;
    p.stages = pl.stages; p.sps = pl.sps;
    p.div_oh = FastDiv((uint32_t)oh);
    p.part_stride = Cout * Cin * KK;
    const dim3 grid((unsigned)(Cin / CT), (unsigned)(Cout / BM), (unsigned)pl.splits);
    const i64 blocks = (i64)grid.x * grid.y * grid.z;
    p.xcd_chunk = blocks % 8 == 0 && blocks <= 0x7fffffff ? (int)(blocks / 8) : 0;
#define FX_WGD_LAUNCH(NKV)                                                                                             \
    case NKV: {                                                                                                        \
        static const hipError_t attr = hipFuncSetAttribute((const void*)wgrad_patch_f64_kernel<NKV>,                   \
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_BUDGET); \
        FX_HIP_CHECK(attr);                                                                                            \
        FX_LAUNCH(grid, dim3(NT), pl.smem, c->stream, (p), wgrad_patch_f64_kernel<NKV>);                                        \
    } break;
    switch (pl.NK) {
        FX_WGD_LAUNCH(3)
        FX_WGD_LAUNCH(4)
        FX_WGD_LAUNCH(7)
        FX_WGD_LAUNCH(8)
        default: FX_REQUIRE(false, "wgrad patch kernel (f64): unexpected row length %d", 8 * pl.NK);
    }
#undef FX_WGD_LAUNCH
    FX_LAUNCH_CHECK();
    const int n = (int)p.part_stride;
    const FastDiv div_row((uint32_t)(KK * Cin)), div_cin((uint32_t)Cin);
    FX_LAUNCH(dim3((unsigned)fx::ceil_div((i64)n, 256)), dim3(256), 0, c->stream, (part, dw, n, pl.splits, (int)Cin, div_row, div_cin), wgrad_f64_reduce_kernel);
    FX_LAUNCH_CHECK();
    return FX_OK;
}

}  // namespace wgd
