// C[M,N] = op(A) . op(B) for small products (f32) in one launch: the layers of a multilayer perceptron at batch 256
// (MatMul::compute / MatMul::gradient, src/ops/matrix.rs:17-55, in the three layouts Linear's forward and backward produce).
//
// The general tiles give such a product too few blocks to fill the chip unless K is split over blocks, and then a second
// kernel adds the partial sums: two launches of 5 to 14 us for a few hundred kFLOP per CU.  Here a block (8 waves) owns a
// 32 x 32 tile of C and splits K over its waves instead: every wave loads its slice of both operands straight from global
// memory into the MFMA operand registers, all loads of the slice in flight at once, and the eight sums are added through LDS in
// wave order -- no LDS staging, no partial sums in memory, one launch.
//
// Operand registers: a group of 8 consecutive k feeds 4 MFMAs; lane l = (i = l % 32, h = l / 32) holds, for MFMA j of the
// group, the element with k = 8 g + 4 h + j of row (column) i.  An operand stored k-contiguous gets that as one 16-byte load,
// one stored row/column-contiguous as four 4-byte loads that run along 128-byte lines.  Both operands use the same assignment,
// so any mix of layouts works.  Elements past K are zeroed in both operands after the load (their addresses are clamped
// into the matrix).
#pragma once
#include <cstdlib>

#include "igemm_core.hpp"

namespace gsmall {
using igemm::f32x16;

constexpr int NT = 512, WAVES = 8, MAXG = 16;  // groups of 8 k per wave: K <= 8 * 8 * 16

struct Params {
    const float* A;
    const float* B;
    float* C;
    const float* bias;  // over n, or null
    int relu;
    int M, N, K;
    int G;       // groups per wave
    int kz;      // K per block when the grid's z dimension splits K (a multiple of 8 * WAVES * G ... see run), else K
    i64 zstride; // elements between the partial results of consecutive z (0 when K is not split)
    float* asum; // optional (K not split): asum[m] = sum over k of op(A)[m][k], written by the first block of every tile row
    const float* mask;  // optional, [M][N] like C (K not split, no bias): C = (op(A) . op(B)) * (mask > 0 ? 1 : 0), fx_relu_bwd's operation
};

// KC: 1 = the operand is stored [rows][K] (k contiguous, K % 4 == 0, 16-byte aligned); 2 = the same layout read element by element
// (any K and alignment: the short reductions of a classifier head's data gradient); 0 = stored [K][rows].
template <int KC>
__device__ __forceinline__ void load_group(const float* __restrict__ base, int row, int rows, int K, int k, float (&v)[4]) {
    if constexpr (KC == 1) {
        const int kc = min(k, K - 4);
        const float4 q = *reinterpret_cast<const float4*>(base + (i64)row * K + kc);
        v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
    } else if constexpr (KC == 2) {
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = base[(i64)row * K + min(k + j, K - 1)];
    } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = base[(i64)min(k + j, K - 1) * rows + row];
    }
}

// The work of one block: tile (bx, by) of the product, range bz of K.  red: WAVES * 16 * 64 floats of LDS, rsum: WAVES * 64.
template <int AKC, int BKC>
__device__ __forceinline__ void small_body(const Params& p, float* red, float* rsum, int bx, int by, int bz) {
    const int tid = threadIdx.x, lane = tid & 63, h = lane >> 5, l32 = lane & 31;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int m0 = by * 32, n0 = bx * 32;
    const int am = min(m0 + l32, p.M - 1), bn = min(n0 + l32, p.N - 1);  // past the edge: a valid row / column, result unused
    const int kbase = bz * p.kz, kend = min(p.K, kbase + p.kz);            // this block's range of K (all of it unless K is split over z)
    const int g0 = wave * p.G;
    const float bias_n = p.bias ? p.bias[bn] : 0.f;  // loaded up front: its latency stays off the closing sum
    float mk[2] = {1.f, 1.f};                        // likewise the mask values of the two elements this lane stores
    if (p.mask) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int e = 2 * wave + u, m = min(m0 + 8 * (e >> 2) + 4 * h + (e & 3), p.M - 1);
            mk[u] = p.mask[(i64)m * p.N + bn];
        }
    }

    float a[MAXG][4], b[MAXG][4];
#pragma unroll
    for (int g = 0; g < MAXG; ++g) {
        if (g < p.G) {  // scalar
            const int k = kbase + 8 * (g0 + g) + 4 * h;
            load_group<AKC>(p.A, am, p.M, p.K, k, a[g]);
            load_group<BKC>(p.B, bn, p.N, p.K, k, b[g]);
        }
    }
    f32x16 acc;
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = 0.f;
    const bool want_asum = p.asum != nullptr && bx == 0;  // block-uniform
    float srow = 0.f;  // this lane's share of the sum of row am of op(A): its k in increasing order
#pragma unroll
    for (int g = 0; g < MAXG; ++g) {
        if (g < p.G) {
            const int k = kbase + 8 * (g0 + g) + 4 * h;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const bool in = k + j < kend;
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(in ? a[g][j] : 0.f, in ? b[g][j] : 0.f, acc, 0, 0, 0);
                if (want_asum) srow = srow + (in ? a[g][j] : 0.f);
            }
        }
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) red[(wave * 16 + e) * 64 + lane] = acc[e];
    if (want_asum) rsum[wave * 64 + lane] = srow;
    __syncthreads();
    if (want_asum && wave == WAVES - 1 && h == 0 && m0 + l32 < p.M) {  // the 16 shares of a row in (wave, half) order
        float v = rsum[l32];
        v = v + rsum[32 + l32];
#pragma unroll
        for (int q = 1; q < WAVES; ++q) {
            v = v + rsum[q * 64 + l32];
            v = v + rsum[q * 64 + 32 + l32];
        }
        p.asum[m0 + l32] = v;
    }
    // wave w finishes accumulator elements 2 w and 2 w + 1: the eight sums in wave order, then the bias kernel's operations
    const int n = n0 + l32;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const int e = 2 * wave + u;
        float v = red[e * 64 + lane];
#pragma unroll
        for (int q = 1; q < WAVES; ++q) v = v + red[(q * 16 + e) * 64 + lane];
        const int m = m0 + 8 * (e >> 2) + 4 * h + (e & 3);
        if (m < p.M && n < p.N) {
            if (p.bias) {
                v = v + bias_n;
                if (p.relu) v = v > 0.f ? v : 0.f;
            }
            if (p.mask) v = v * (mk[u] > 0.f ? 1.f : 0.f);
            p.C[(i64)bz * p.zstride + (i64)m * p.N + n] = v;
        }
    }
}

template <int AKC, int BKC>
__global__ __launch_bounds__(NT) void small_kernel(const Params p) {
    __shared__ float red[WAVES * 16 * 64];
    __shared__ float rsum[WAVES * 64];
    small_body<AKC, BKC>(p, red, rsum, blockIdx.x, blockIdx.y, blockIdx.z);
}

// Two independent products in one launch, blockIdx.z picks the product (neither splits K): the data and the weight gradient of a
// Linear layer, dX = dY . W (both operands as stored: A k-contiguous) and dW = dY^T . X (A stored [K, M]).  A block outside its
// product's tile range leaves at once.
template <int A0>  // how the first product reads its A: 1 or 2
__global__ __launch_bounds__(NT) void small_pair_kernel(const Params p0, const Params p1) {
    __shared__ float red[WAVES * 16 * 64];
    __shared__ float rsum[WAVES * 64];
    const int bx = blockIdx.x, by = blockIdx.y;
    if (blockIdx.z == 0) {
        if (bx * 32 < p0.N && by * 32 < p0.M) small_body<A0, 0>(p0, red, rsum, bx, by, 0);
    } else {
        if (bx * 32 < p1.N && by * 32 < p1.M) small_body<0, 0>(p1, red, rsum, bx, by, 0);
    }
}

// ---- 16 x 16 tiles (f32) on v_mfma_f32_16x16x4_f32 -----------------------------------------------------------------------------
// A product of a few dozen 32 x 32 tiles leaves most of the chip idle and every block with a long operand read ([256,784] x
// [784,256]: 64 blocks of 200 KB each).  With 16 x 16 tiles there are four times the blocks at half the bytes each.  A group of
// 16 consecutive k feeds 4 MFMAs; lane l = (i = l % 16, q = l / 16) holds, for MFMA j of the group, the element with
// k = 16 g + 4 q + j of row (column) i -- the same 16-byte load per lane as in the 32 x 32 kernel -- and 4 of the 256 sums
// (row 4 q + e, column i).  K is split over the 8 waves and added through LDS in wave order as above.
typedef float f32x4 __attribute__((ext_vector_type(4)));
constexpr int MAXG16 = 16;  // groups of 16 k per wave: K <= 16 * 8 * 16

template <int AKC, int BKC>
__global__ __launch_bounds__(NT) void small16_kernel(const Params p) {
    __shared__ float red[WAVES * 4 * 64];
    const int tid = threadIdx.x, lane = tid & 63, q = lane >> 4, i = lane & 15;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int m0 = blockIdx.y * 16, n0 = blockIdx.x * 16;
    const int am = min(m0 + i, p.M - 1), bn = min(n0 + i, p.N - 1);  // past the edge: a valid row / column, result unused
    const int g0 = wave * p.G;
    const float bias_n = p.bias ? p.bias[bn] : 0.f;

    float a[MAXG16][4], b[MAXG16][4];
#pragma unroll
    for (int g = 0; g < MAXG16; ++g) {
        if (g < p.G) {  // scalar
            const int k = 16 * (g0 + g) + 4 * q;
            load_group<AKC>(p.A, am, p.M, p.K, k, a[g]);
            load_group<BKC>(p.B, bn, p.N, p.K, k, b[g]);
        }
    }
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int g = 0; g < MAXG16; ++g) {
        if (g < p.G) {
            const int k = 16 * (g0 + g) + 4 * q;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const bool in = k + j < p.K;
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(in ? a[g][j] : 0.f, in ? b[g][j] : 0.f, acc, 0, 0, 0);
            }
        }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) red[(wave * 4 + e) * 64 + lane] = acc[e];
    __syncthreads();
    // waves 0 .. 3 finish accumulator element `wave`: the eight sums in wave order, then the bias kernel's operations
    if (wave < 4) {
        const int e = wave;
        float v = red[e * 64 + lane];
#pragma unroll
        for (int w = 1; w < WAVES; ++w) v = v + red[(w * 4 + e) * 64 + lane];
        const int m = m0 + 4 * q + e, n = n0 + i;
        if (m < p.M && n < p.N) {
            if (p.bias) {
                v = v + bias_n;
                if (p.relu) v = v > 0.f ? v : 0.f;
            }
            p.C[(i64)m * p.N + n] = v;
        }
    }
}

// ---- f64 twin on v_mfma_f64_16x16x4_f64 -------------------------------------------------------------------------------------
// The 32 x 32 tile is 2 x 2 MFMA blocks of 16 x 16; a group of 8 consecutive k feeds 2 MFMA steps of 4 k each.  Lane
// l = (i = l % 16, q = l / 16) holds, for step j of the group, the element with k = 8 g + 2 q + j of rows (columns) i and i + 16:
// one 16-byte load per row for a k-contiguous operand, two 8-byte loads along 128-byte lines otherwise.  A wave keeps at most
// MAXG_D groups in flight (128 registers) and walks its slice of K in batches of that size.
using igemm::f64x4;
constexpr int MAXG_D = 8;

struct ParamsD {
    const double* A;
    const double* B;
    double* C;
    const double* bias;
    int relu;
    int M, N, K;
    int G;  // groups per wave
    int kz;
    i64 zstride;
    double* asum;        // optional, as in Params
    const double* mask;  // optional, as in Params
};

template <int KC>
__device__ __forceinline__ void load_group_d(const double* __restrict__ base, int row, int rows, int K, int k, double (&v)[2]) {
    if constexpr (KC == 1) {
        typedef double d2 __attribute__((ext_vector_type(2)));
        const d2 q = *reinterpret_cast<const d2*>(base + (i64)row * K + min(k, K - 2));
        v[0] = q.x; v[1] = q.y;
    } else if constexpr (KC == 2) {
#pragma unroll
        for (int j = 0; j < 2; ++j) v[j] = base[(i64)row * K + min(k + j, K - 1)];
    } else {
#pragma unroll
        for (int j = 0; j < 2; ++j) v[j] = base[(i64)min(k + j, K - 1) * rows + row];
    }
}

// red_d: [8 waves][16 elements][64 lanes] doubles of LDS
template <int AKC, int BKC>
__device__ __forceinline__ void small_body_f64(const ParamsD& p, double* red_d, int bx, int by, int bz) {
    const int tid = threadIdx.x, lane = tid & 63, q = lane >> 4, l16 = lane & 15;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int m0 = by * 32, n0 = bx * 32;
    const int am0 = min(m0 + l16, p.M - 1), am1 = min(m0 + 16 + l16, p.M - 1);  // past the edge: a valid row / column, result unused
    const int bn0 = min(n0 + l16, p.N - 1), bn1 = min(n0 + 16 + l16, p.N - 1);
    const int kbase = bz * p.kz, kend = min(p.K, kbase + p.kz);
    const int g0 = wave * p.G;
    // this wave finishes the column block (wave / 2) % 2 in the closing sum; its bias is loaded up front
    const double bias_n = p.bias ? p.bias[(wave >> 1) & 1 ? bn1 : bn0] : 0.;
    double mk[2] = {1., 1.};  // the mask values of the two elements this lane stores
    if (p.mask) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int el = 2 * wave + u, blk = el >> 2, e = el & 3;
            const int m = min(m0 + 16 * (blk >> 1) + 4 * e + q, p.M - 1);
            mk[u] = p.mask[(i64)m * p.N + ((blk & 1) ? bn1 : bn0)];
        }
    }
    f64x4 acc[2][2];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[a][b][e] = 0.;
    const bool want_asum = p.asum != nullptr && bx == 0;  // block-uniform
    double srow0 = 0., srow1 = 0.;  // this lane's shares of the sums of rows am0 and am1 of op(A): its k in increasing order
    for (int gb = 0; gb < p.G; gb += MAXG_D) {  // scalar loop: batches of MAXG_D groups
        double a0[MAXG_D][2], a1[MAXG_D][2], b0[MAXG_D][2], b1[MAXG_D][2];
#pragma unroll
        for (int g = 0; g < MAXG_D; ++g) {
            if (gb + g < p.G) {
                const int k = kbase + 8 * (g0 + gb + g) + 2 * q;
                load_group_d<AKC>(p.A, am0, p.M, p.K, k, a0[g]);
                load_group_d<AKC>(p.A, am1, p.M, p.K, k, a1[g]);
                load_group_d<BKC>(p.B, bn0, p.N, p.K, k, b0[g]);
                load_group_d<BKC>(p.B, bn1, p.N, p.K, k, b1[g]);
            }
        }
#pragma unroll
        for (int g = 0; g < MAXG_D; ++g) {
            if (gb + g < p.G) {
                const int k = kbase + 8 * (g0 + gb + g) + 2 * q;
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const bool in = k + j < kend;  // past K: zeros in both operands, whatever the clamped loads returned
                    const double x0 = in ? a0[g][j] : 0., x1 = in ? a1[g][j] : 0., y0 = in ? b0[g][j] : 0., y1 = in ? b1[g][j] : 0.;
                    acc[0][0] = __builtin_amdgcn_mfma_f64_16x16x4f64(x0, y0, acc[0][0], 0, 0, 0);
                    acc[0][1] = __builtin_amdgcn_mfma_f64_16x16x4f64(x0, y1, acc[0][1], 0, 0, 0);
                    acc[1][0] = __builtin_amdgcn_mfma_f64_16x16x4f64(x1, y0, acc[1][0], 0, 0, 0);
                    acc[1][1] = __builtin_amdgcn_mfma_f64_16x16x4f64(x1, y1, acc[1][1], 0, 0, 0);
                    if (want_asum) { srow0 = srow0 + x0; srow1 = srow1 + x1; }
                }
            }
        }
    }
    // element index 4 (2 a + b) + e of lane l is C[m0 + 16 a + 4 e + l / 16][n0 + 16 b + l % 16]
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int e = 0; e < 4; ++e) red_d[(wave * 16 + 4 * (2 * a + b) + e) * 64 + lane] = acc[a][b][e];
    __syncthreads();
    // wave w finishes elements 2 w and 2 w + 1: the eight sums in wave order, then the bias kernel's operations
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const int el = 2 * wave + u, blk = el >> 2, e = el & 3;
        double v = red_d[el * 64 + lane];
#pragma unroll
        for (int w = 1; w < WAVES; ++w) v = v + red_d[(w * 16 + el) * 64 + lane];
        const int m = m0 + 16 * (blk >> 1) + 4 * e + q, n = n0 + 16 * (blk & 1) + l16;
        if (m < p.M && n < p.N) {
            if (p.bias) {
                v = v + bias_n;
                if (p.relu) v = v > 0. ? v : 0.;
            }
            if (p.mask) v = v * (mk[u] > 0. ? 1. : 0.);
            p.C[(i64)bz * p.zstride + (i64)m * p.N + n] = v;
        }
    }
    if (want_asum) {  // block-uniform: the row sums go through the same LDS once the closing sum has read it
        __syncthreads();
        red_d[(wave * 2 + 0) * 64 + lane] = srow0;
        red_d[(wave * 2 + 1) * 64 + lane] = srow1;
        __syncthreads();
        if (wave == WAVES - 1 && lane < 32 && m0 + lane < p.M) {  // row m0 + lane: its 32 shares in (wave, quarter) order
            const int r = lane >> 4, i = lane & 15;
            double v = 0.;
#pragma unroll
            for (int w = 0; w < WAVES; ++w)
#pragma unroll
                for (int qq = 0; qq < 4; ++qq) {
                    const double t = red_d[(w * 2 + r) * 64 + qq * 16 + i];
                    v = (w == 0 && qq == 0) ? t : v + t;
                }
            p.asum[m0 + lane] = v;
        }
    }
}

template <int AKC, int BKC>
__global__ __launch_bounds__(NT) void small_kernel_f64(const ParamsD p) {
    FX_DYNAMIC_SMEM(double, red_d);
    small_body_f64<AKC, BKC>(p, red_d, blockIdx.x, blockIdx.y, blockIdx.z);
}

template <int A0>
__global__ __launch_bounds__(NT) void small_pair_kernel_f64(const ParamsD p0, const ParamsD p1) {  // as small_pair_kernel
    FX_DYNAMIC_SMEM(double, red_d);
    const int bx = blockIdx.x, by = blockIdx.y;
    if (blockIdx.z == 0) {
        if (bx * 32 < p0.N && by * 32 < p0.M) small_body_f64<A0, 0>(p0, red_d, bx, by, 0);
    } else {
        if (bx * 32 < p1.N && by * 32 < p1.M) small_body_f64<0, 0>(p1, red_d, bx, by, 0);
    }
}

// How a product runs here: K in one block (splits == 1), or split over the grid's z dimension into `splits` ranges of kz whose
// partial results the caller adds in order (igemm::launch_splitk_reduce) -- long reductions with few tiles, the forward product of
// a classifier head ([256,16384] x [16384,10]).
struct Plan {
    bool ok = false;
    int G = 0, kz = 0, splits = 1;
    bool a_elems = false;  // A is k-contiguous but not readable in 16-byte pieces (K % 4, alignment): element loads
    bool tile16 = false;   // f32: 16 x 16 tiles (few 32 x 32 tiles and a long enough reduction); no row sums or mask in this form
};

// allow16: the caller wants neither row sums nor a mask nor a pair launch (those exist for 32 x 32 tiles only)
template <typename T>
inline Plan make_plan(int num_cus, bool ta, bool tb, i64 M, i64 N, i64 K, const T* A, const T* B, bool allow16 = false) {
    Plan pl;
    constexpr int KV = 16 / (int)sizeof(T);  // elements per 16-byte load of a k-contiguous operand
    if (K < 1 || M < 1 || N < 1 || K >= (1ll << 30)) return pl;
    if (K < 32 && ta) return pl;  // short reductions: only with a k-contiguous A, read element by element (the general tiles serve the others)
    if (!ta && (K % KV != 0 || !fx::aligned16(A) || K < 32)) pl.a_elems = true;
    if (tb && (K % KV != 0 || !fx::aligned16(B))) return pl;
    const i64 tiles = fx::ceil_div(M, (i64)32) * fx::ceil_div(N, (i64)32);
    // a 32 x 32 tile re-reads each operand once per tile row / column: M N K sizeof(T) / 16 bytes through L2, kept under 32 MB (f32) / 64 MB (f64)
    if (tiles > 2 * (i64)num_cus || M * N * K > (1ll << 27)) return pl;
    const i64 kmax = 8 * WAVES * MAXG;  // the most one block takes
    if (K <= kmax) {
        pl.G = (int)fx::ceil_div(fx::ceil_div(K, (i64)8), (i64)WAVES);
        pl.kz = (int)K;
        if constexpr (sizeof(T) == 4) {
            // fewer 32 x 32 tiles than half the CUs, each reading K >= 128 deep: 16 x 16 tiles fill more of the chip
            const i64 tiles16 = fx::ceil_div(M, (i64)16) * fx::ceil_div(N, (i64)16);
            if (allow16 && !pl.a_elems && 2 * tiles < (i64)num_cus && tiles16 <= 2 * (i64)num_cus && K >= 128 && N >= 16) {
                pl.tile16 = true;
                pl.G = (int)fx::ceil_div(fx::ceil_div(K, (i64)16), (i64)WAVES);
            }
        }
    } else {
        // split K over blocks: about 2 blocks per CU, each at least 256 deep, ranges a multiple of 8 * WAVES
        if (M * N > (1 << 18)) return pl;  // the partial sums stay small
        i64 splits = std::max<i64>(fx::ceil_div(K, kmax), std::min<i64>(2 * (i64)num_cus / tiles, K / 256));
        i64 kz = fx::ceil_div(fx::ceil_div(K, splits), (i64)(8 * WAVES)) * (8 * WAVES);
        splits = fx::ceil_div(K, kz);
        if (kz > kmax || splits > 65535) return pl;
        pl.G = (int)(kz / (8 * WAVES));
        pl.kz = (int)kz;
        pl.splits = (int)splits;
    }
    pl.ok = true;
    return pl;
}

template <typename T> inline i64 workspace_bytes(const Plan& pl, i64 M, i64 N) { return pl.splits > 1 ? (i64)pl.splits * M * N * (i64)sizeof(T) : 0; }

// part: workspace_bytes() of scratch when pl.splits > 1 (the caller then adds the partial results, with the bias)
// asum (optional, only with pl.splits == 1): receives the row sums of op(A)
inline int run_f64(fx_ctx* c, const Plan& pl, bool ta, bool tb, i64 M, i64 N, i64 K, const double* A, const double* B, double* C, const double* bias,
                   int relu, double* part, double* asum = nullptr) {
    const bool split = pl.splits > 1;
    FX_REQUIRE(!(split && asum), "small product: row sums need an unsplit reduction");
    ParamsD p{A, B, split ? part : C, split ? nullptr : bias, relu, (int)M, (int)N, (int)K, pl.G, pl.kz, split ? M * N : 0, asum, nullptr};
    const dim3 grid((unsigned)fx::ceil_div(N, (i64)32), (unsigned)fx::ceil_div(M, (i64)32), (unsigned)pl.splits);
    const size_t lds = (size_t)WAVES * 16 * 64 * sizeof(double);
    if (!ta && pl.a_elems && !tb) FX_LAUNCH(grid, dim3(NT), lds, c->stream, (p), small_kernel_f64<2, 0>);
    else if (!ta && pl.a_elems) FX_LAUNCH(grid, dim3(NT), lds, c->stream, (p), small_kernel_f64<2, 1>);
    else if (!ta && !tb) FX_LAUNCH(grid, dim3(NT), lds, c->stream, (p), small_kernel_f64<1, 0>);
    else if (!ta && tb) FX_LAUNCH(grid, dim3(NT), lds, c->stream, (p), small_kernel_f64<1, 1>);
    else if (ta && !tb) FX_LAUNCH(grid, dim3(NT), lds, c->stream, (p), small_kernel_f64<0, 0>);
    else FX_LAUNCH(grid, dim3(NT), lds, c->stream, (p), small_kernel_f64<0, 1>);
    FX_LAUNCH_CHECK();
    return FX_OK;
}

inline int run(fx_ctx* c, const Plan& pl, bool ta, bool tb, i64 M, i64 N, i64 K, const float* A, const float* B, float* C, const float* bias, int relu,
               float* part, float* asum = nullptr) {
    const bool split = pl.splits > 1;
    FX_REQUIRE(!(split && asum), "small product: row sums need an unsplit reduction");
    Params p{A, B, split ? part : C, split ? nullptr : bias, relu, (int)M, (int)N, (int)K, pl.G, pl.kz, split ? M * N : 0, asum, nullptr};
    if (pl.tile16) {
        FX_REQUIRE(!split && !asum && !pl.a_elems, "small product: 16 x 16 tiles take neither a split K nor row sums");
        const dim3 grid16((unsigned)fx::ceil_div(N, (i64)16), (unsigned)fx::ceil_div(M, (i64)16));
        if (!ta && !tb) FX_LAUNCH(grid16, dim3(NT), 0, c->stream, (p), small16_kernel<1, 0>);
        else if (!ta && tb) FX_LAUNCH(grid16, dim3(NT), 0, c->stream, (p), small16_kernel<1, 1>);
        else if (ta && !tb) FX_LAUNCH(grid16, dim3(NT), 0, c->stream, (p), small16_kernel<0, 0>);
        else FX_LAUNCH(grid16, dim3(NT), 0, c->stream, (p), small16_kernel<0, 1>);
        FX_LAUNCH_CHECK();
        return FX_OK;
    }
    const dim3 grid((unsigned)fx::ceil_div(N, (i64)32), (unsigned)fx::ceil_div(M, (i64)32), (unsigned)pl.splits);
    if (!ta && pl.a_elems && !tb) FX_LAUNCH(grid, dim3(NT), 0, c->stream, (p), small_kernel<2, 0>);
    else if (!ta && pl.a_elems) FX_LAUNCH(grid, dim3(NT), 0, c->stream, (p), small_kernel<2, 1>);
    else if (!ta && !tb) FX_LAUNCH(grid, dim3(NT), 0, c->stream, (p), small_kernel<1, 0>);
    else if (!ta && tb) FX_LAUNCH(grid, dim3(NT), 0, c->stream, (p), small_kernel<1, 1>);
    else if (ta && !tb) FX_LAUNCH(grid, dim3(NT), 0, c->stream, (p), small_kernel<0, 0>);
    else FX_LAUNCH(grid, dim3(NT), 0, c->stream, (p), small_kernel<0, 1>);
    FX_LAUNCH_CHECK();
    return FX_OK;
}

// dX[M0,N0] = A0 . B0 (A0 stored [M0,K0], B0 stored [K0,N0]) and dW[M1,N1] = A1^T . B1 (A1 stored [K1,M1], B1 stored [K1,N1]) in one
// launch; both plans unsplit.  asum1 (optional): the row sums of A1^T, i.e. the column sums of A1.
// mask0 (optional, [M0][N0]): the first product is stored times (mask0 > 0 ? 1 : 0).
inline int run_pair(fx_ctx* c, const Plan& p0, const Plan& p1, i64 M0, i64 N0, i64 K0, const float* A0, const float* B0, float* C0, i64 M1, i64 N1,
                    i64 K1, const float* A1, const float* B1, float* C1, float* asum1, const float* mask0) {
    FX_REQUIRE(p0.splits == 1 && p1.splits == 1, "small product pair: unsplit reductions only");
    Params a{A0, B0, C0, nullptr, 0, (int)M0, (int)N0, (int)K0, p0.G, p0.kz, 0, nullptr, mask0};
    Params b{A1, B1, C1, nullptr, 0, (int)M1, (int)N1, (int)K1, p1.G, p1.kz, 0, asum1, nullptr};
    const dim3 grid((unsigned)fx::ceil_div(std::max(N0, N1), (i64)32), (unsigned)fx::ceil_div(std::max(M0, M1), (i64)32), 2);
    if (p0.a_elems) FX_LAUNCH(grid, dim3(NT), 0, c->stream, (a, b), small_pair_kernel<2>);
    else FX_LAUNCH(grid, dim3(NT), 0, c->stream, (a, b), small_pair_kernel<1>);
    FX_LAUNCH_CHECK();
    return FX_OK;
}
inline int run_pair(fx_ctx* c, const Plan& p0, const Plan& p1, i64 M0, i64 N0, i64 K0, const double* A0, const double* B0, double* C0, i64 M1,
                    i64 N1, i64 K1, const double* A1, const double* B1, double* C1, double* asum1, const double* mask0) {
    FX_REQUIRE(p0.splits == 1 && p1.splits == 1, "small product pair: unsplit reductions only");
    ParamsD a{A0, B0, C0, nullptr, 0, (int)M0, (int)N0, (int)K0, p0.G, p0.kz, 0, nullptr, mask0};
    ParamsD b{A1, B1, C1, nullptr, 0, (int)M1, (int)N1, (int)K1, p1.G, p1.kz, 0, asum1, nullptr};
    const dim3 grid((unsigned)fx::ceil_div(std::max(N0, N1), (i64)32), (unsigned)fx::ceil_div(std::max(M0, M1), (i64)32), 2);
    const size_t lds = (size_t)WAVES * 16 * 64 * sizeof(double);
    if (p0.a_elems) FX_LAUNCH(grid, dim3(NT), lds, c->stream, (a, b), small_pair_kernel_f64<2>);
    else FX_LAUNCH(grid, dim3(NT), lds, c->stream, (a, b), small_pair_kernel_f64<1>);
    FX_LAUNCH_CHECK();
    return FX_OK;
}

}  // namespace gsmall
