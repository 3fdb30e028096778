// TEST INFRASTRUCTURE ONLY (part of the CPU oracle; never linked into the product library).
//
// Single-thread cache-blocked GEMM used wherever the Ferrox CPU backend calls ndarray's `dot`
// (src/backend/storage/cpu.rs:999, src/backend/storage/extensions/convolutions.rs:256, 296, 332).
// ndarray 0.16.1 forwards those calls to matrixmultiply 0.3.10 (Cargo.lock), a packed, register-blocked
// single-thread SIMD kernel whose source is not part of the reference tree.  This file restates that
// published algorithm shape (pack A into MR-row panels, B into NR-column panels, k-blocked micro-kernel
// with fused multiply-add) so that the CPU baseline is not penalised by a naive triple loop.
// The summation ORDER of matrixmultiply is not reproduced: results are compared by tolerance only.
#include <cstdint>
#include <cstring>
#include <vector>
#include <algorithm>

typedef int64_t i64;

namespace {

template <typename T> struct Vec;
template <> struct Vec<float> { typedef float type __attribute__((vector_size(32))); static constexpr int W = 8; };
template <> struct Vec<double> { typedef double type __attribute__((vector_size(32))); static constexpr int W = 4; };

constexpr int MR = 6;

template <typename T>
inline void micro_kernel(i64 kc, const T* __restrict Ap, const T* __restrict Bp, T* __restrict C, i64 ldc, int mr,
                         int nr) {
    typedef typename Vec<T>::type V;
    constexpr int W = Vec<T>::W;
    constexpr int NR = 2 * W;
    V acc[MR][2];
    for (int i = 0; i < MR; ++i) { acc[i][0] = V{} ; acc[i][1] = V{}; }
    for (i64 k = 0; k < kc; ++k) {
        V b0, b1;
        std::memcpy(&b0, Bp + k * NR, sizeof(V));
        std::memcpy(&b1, Bp + k * NR + W, sizeof(V));
        const T* a = Ap + k * MR;
#pragma GCC unroll 6
        for (int i = 0; i < MR; ++i) {
            const T ai = a[i];
            V av;
            for (int w = 0; w < W; ++w) av[w] = ai;
            acc[i][0] += av * b0;
            acc[i][1] += av * b1;
        }
    }
    if (mr == MR && nr == NR) {
        for (int i = 0; i < MR; ++i) {
            V c0, c1;
            std::memcpy(&c0, C + i * ldc, sizeof(V));
            std::memcpy(&c1, C + i * ldc + W, sizeof(V));
            c0 += acc[i][0];
            c1 += acc[i][1];
            std::memcpy(C + i * ldc, &c0, sizeof(V));
            std::memcpy(C + i * ldc + W, &c1, sizeof(V));
        }
    } else {
        for (int i = 0; i < mr; ++i)
            for (int j = 0; j < nr; ++j) C[i * ldc + j] += (j < W ? acc[i][0][j] : acc[i][1][j - W]);
    }
}

template <typename T>
void gemm_nn(i64 M, i64 N, i64 K, const T* A, i64 lda, const T* B, i64 ldb, T* C, i64 ldc) {
    constexpr int W = Vec<T>::W;
    constexpr int NR = 2 * W;
    const i64 KC = 256, MC = 96, NC = 4096;
    for (i64 m = 0; m < M; ++m) std::memset(C + m * ldc, 0, sizeof(T) * N);
    std::vector<T> Bp((size_t)(KC * (NC + NR))), Ap((size_t)(KC * (MC + MR)));
    for (i64 jj = 0; jj < N; jj += NC) {
        const i64 nc = std::min(NC, N - jj);
        for (i64 kk = 0; kk < K; kk += KC) {
            const i64 kc = std::min(KC, K - kk);
            // pack B[kk:kk+kc, jj:jj+nc] into NR-wide panels
            for (i64 j = 0; j < nc; j += NR) {
                const int nr = (int)std::min<i64>(NR, nc - j);
                T* dst = Bp.data() + (j / NR) * (kc * NR);
                for (i64 k = 0; k < kc; ++k) {
                    const T* src = B + (kk + k) * ldb + jj + j;
                    int c = 0;
                    for (; c < nr; ++c) dst[k * NR + c] = src[c];
                    for (; c < NR; ++c) dst[k * NR + c] = T(0);
                }
            }
            for (i64 ii = 0; ii < M; ii += MC) {
                const i64 mc = std::min(MC, M - ii);
                for (i64 i = 0; i < mc; i += MR) {
                    const int mr = (int)std::min<i64>(MR, mc - i);
                    T* dst = Ap.data() + (i / MR) * (kc * MR);
                    for (i64 k = 0; k < kc; ++k) {
                        int r = 0;
                        for (; r < mr; ++r) dst[k * MR + r] = A[(ii + i + r) * lda + kk + k];
                        for (; r < MR; ++r) dst[k * MR + r] = T(0);
                    }
                }
                for (i64 j = 0; j < nc; j += NR) {
                    const int nr = (int)std::min<i64>(NR, nc - j);
                    for (i64 i = 0; i < mc; i += MR) {
                        const int mr = (int)std::min<i64>(MR, mc - i);
                        micro_kernel<T>(kc, Ap.data() + (i / MR) * (kc * MR), Bp.data() + (j / NR) * (kc * NR),
                                        C + (ii + i) * ldc + jj + j, ldc, mr, nr);
                    }
                }
            }
        }
    }
}

template <typename T>
std::vector<T> transposed(const T* X, i64 rows, i64 cols) {  // X is [rows, cols] -> returns [cols, rows]
    std::vector<T> t((size_t)(rows * cols));
    const i64 BS = 32;
    for (i64 r0 = 0; r0 < rows; r0 += BS)
        for (i64 c0 = 0; c0 < cols; c0 += BS)
            for (i64 r = r0; r < std::min(rows, r0 + BS); ++r)
                for (i64 c = c0; c < std::min(cols, c0 + BS); ++c) t[(size_t)(c * rows + r)] = X[r * cols + c];
    return t;
}

}  // namespace

// C[M,N] = op(A) . op(B);  ta: A is stored [K,M];  tb: B is stored [N,K].
template <typename T>
void orc_gemm_fast(int ta, int tb, i64 M, i64 N, i64 K, const T* A, const T* B, T* C) {
    std::vector<T> At, Bt;
    if (ta) { At = transposed(A, K, M); A = At.data(); }
    if (tb) { Bt = transposed(B, N, K); B = Bt.data(); }
    gemm_nn<T>(M, N, K, A, K, B, N, C, N);
}
template void orc_gemm_fast<float>(int, int, i64, i64, i64, const float*, const float*, float*);
template void orc_gemm_fast<double>(int, int, i64, i64, i64, const double*, const double*, double*);
