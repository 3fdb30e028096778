// C[M,N] = A^T . B for a thin product (f32): A stored [K,M] with at most 32 columns, B stored [K,N], a short reduction
// (K up to about 2000) and a wide N -- the weight gradient of a classifier head, dW[out,in] = dY^T[out,batch] . X[batch,in]
// (MatMul::gradient, src/ops/matrix.rs:34-55, as Linear's backward calls it).
//
// The product reads B once and is bound by that read; the general tiles stage it through LDS in 16-deep slabs and split K
// over blocks with a second kernel for the sum.  Here a block (8 waves) takes 64 columns of N over the whole of K: A goes to
// LDS once (zero padded to 32 columns), every wave owns 32 columns x a quarter of K and feeds the MFMA B operand straight from
// global memory (lane l holds B[k + l / 32][n + l % 32], so a load instruction reads two 128-byte runs), 32 loads in flight per
// lane.  The four quarters of K are added through LDS in a fixed order: one launch, no partial sums in memory.
// (16-byte loads with four accumulator blocks per wave and 128 columns per block measured slower: 12.4 against 9.8 us at
// [10,256] x [256,16384]; the MFMA rows past M are idle either way.)
#pragma once
#include <cstdlib>

#include "igemm_core.hpp"

namespace gthin {
using igemm::f32x16;

constexpr int NT = 512, U = 16, BN = 64, KQ = 4;
constexpr size_t LDS_LIMIT = 160 * 1024;

struct Params {
    const float* A;
    const float* B;
    float* C;
    const float* bias;  // over n, or null
    int relu;
    int M, N, K;
    int as_rows;  // rows of A in LDS: the rows of K, zero padded to what the padded rounds of the last quarter index
    float* asum;  // optional: asum[m] = sum over k of A[k][m], written by the first block
};

__global__ __launch_bounds__(NT) void thin_tn_kernel(const Params p) {
    FX_DYNAMIC_SMEM(float, smem);
    float* red = smem;                          // [3 quarters][2 column slabs][16][64]
    float* As = smem + (KQ - 1) * 2 * 16 * 64;  // [as_rows][32]: A[k][m], zero for m >= M and k >= K
    const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5, l32 = lane & 31;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int cs = wave & 1, kq = wave >> 1;
    const int n = blockIdx.x * BN + cs * 32 + l32, nc = min(n, p.N - 1);  // past the last column: a valid address, value unused
    const int pairs = (p.K + 1) >> 1, pq = (pairs + KQ - 1) / KQ;         // pairs of rows of K; pairs per quarter
    const int p_beg = kq * pq, p_end = min(pairs, p_beg + pq);
    const float* bcol = p.B + nc;
    const float bias_n = p.bias ? p.bias[nc] : 0.f;  // loaded up front: its latency stays off the closing sum

    float b[2][U];
    auto load = [&](int set, int p0) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int r = min(2 * (p0 + u) + half, p.K - 1);  // unconditional loads (rows past the end re-read the last one)
            b[set][u] = bcol[(i64)r * p.N];
        }
    };
    load(0, p_beg);  // in flight while A is staged
    load(1, p_beg + U);
    // A[k][m] -> As[k][m], zeros elsewhere; eight gathers in flight per thread
    const int total = p.as_rows * 32;
    for (int i0 = tid; i0 < total; i0 += 8 * NT) {
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int i = i0 + j * NT, k = i >> 5, m = i & 31;
            const bool in = i < total && k < p.K && m < p.M;
            v[j] = p.A[in ? k * p.M + m : 0];
            if (!in) v[j] = 0.f;
        }
#pragma unroll
        for (int j = 0; j < 8; ++j)
            if (i0 + j * NT < total) As[i0 + j * NT] = v[j];
    }
    __syncthreads();
    const bool want_asum = p.asum != nullptr && blockIdx.x == 0;  // block-uniform
    float* rs = As + p.as_rows * 32;                              // [16 parts][32 columns]
    if (want_asum) {  // column m of A from LDS: part q adds rows q, q + 16, ... (rows past K are zero)
        const int m = tid & 31, part = tid >> 5;
        float v = 0.f;
        for (int k = part; k < p.as_rows; k += 16) v = v + As[k * 32 + m];
        rs[part * 32 + m] = v;
    }

    f32x16 acc;
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = 0.f;
    const float* a = As + half * 32 + l32;
    auto mma = [&](int set, int p0) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const bool in = p0 + u < p_end && 2 * (p0 + u) + half < p.K;  // past the end of this quarter: a zero, whatever was loaded
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[(p0 + u) * 64], in ? b[set][u] : 0.f, acc, 0, 0, 0);
        }
    };
    // rounds of 2 U pairs; the loads of the round after are issued as soon as a register set is free.  Pairs past the end of
    // this quarter multiply zeros (and their rows of A in LDS are zero).
    const int rounds = (p_end - p_beg + 2 * U - 1) / (2 * U);
    int p0 = p_beg;
    for (int r = 0; r < rounds; ++r, p0 += 2 * U) {
        mma(0, p0);
        if (r + 1 < rounds) load(0, p0 + 2 * U);
        mma(1, p0 + U);
        if (r + 1 < rounds) load(1, p0 + 3 * U);
    }

    if (kq != 0) {
#pragma unroll
        for (int e = 0; e < 16; ++e) red[(((kq - 1) * 2 + cs) * 16 + e) * 64 + lane] = acc[e];
    }
    __syncthreads();
    if (want_asum && wave == 7 && lane < p.M) {  // the 16 parts in order
        float v = rs[lane];
#pragma unroll
        for (int q = 1; q < 16; ++q) v = v + rs[q * 32 + lane];
        p.asum[lane] = v;
    }
    if (kq == 0 && n < p.N) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const int m = igemm::Mfma<float>::row(e, lane);
            if (m < p.M) {
                float v = acc[e];
#pragma unroll
                for (int q = 0; q < KQ - 1; ++q) v = v + red[((q * 2 + cs) * 16 + e) * 64 + lane];
                if (p.bias) {  // the operations of the bias kernel, in its order
                    v = v + bias_n;
                    if (p.relu) v = v > 0.f ? v : 0.f;
                }
                p.C[(i64)m * p.N + n] = v;
            }
        }
    }
}

inline int as_rows(i64 K) {
    const i64 pairs = (K + 1) / 2, pq = (pairs + KQ - 1) / KQ;
    return (int)(2 * ((KQ - 1) * pq + (pq + 2 * U - 1) / (2 * U) * (2 * U)));
}
inline size_t lds_bytes(i64 K) { return ((size_t)as_rows(K) * 32 + (KQ - 1) * 2 * 16 * 64 + 16 * 32) * sizeof(float); }

// TN products this kernel takes: the general path needs two launches (split K) and stages B in 64-byte pieces.
inline bool eligible(int num_cus, bool ta, bool tb, i64 M, i64 N, i64 K) {
    return ta && !tb && M >= 1 && M <= 32 && K >= 32 && K <= 2048 && lds_bytes(K) <= LDS_LIMIT && N >= 32 * (i64)num_cus &&
           N < (1ll << 31) - BN;
}

inline int run(fx_ctx* c, i64 M, i64 N, i64 K, const float* A, const float* B, float* C, const float* bias, int relu, float* asum = nullptr) {
    Params p{A, B, C, bias, relu, (int)M, (int)N, (int)K, as_rows(K), asum};
    static const hipError_t attr = hipFuncSetAttribute((const void*)thin_tn_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_LIMIT);
    FX_HIP_CHECK(attr);
    FX_LAUNCH(dim3((unsigned)fx::ceil_div(N, (i64)BN)), dim3(NT), lds_bytes(K), c->stream, (p), thin_tn_kernel);
    FX_LAUNCH_CHECK();
    return FX_OK;
}

}  // namespace gthin
