// fx_gemm: C[M,N] = op(A) . op(B) on the MFMA pipes (f32: v_mfma_f32_32x32x2_f32, f64: v_mfma_f64_16x16x4_f64).
// Replaces kernels/matmul.cu (16x16 shared-memory tiles, 75 % of threads idle) and serves MatMul::compute /
// MatMul::gradient (src/ops/matrix.rs:17-55) without materialised transposes via the trans flags.
// Small or skinny products are split along K into deterministic partial sums (no atomics).
#include <cstdlib>

#include "gemm_lds.hpp"
#include "gemm_thin.hpp"
#include "gemm_small.hpp"

extern "C" int fx_bias_act_f32(fx_ctx*, float*, const float*, int64_t, int64_t, int64_t, int);
extern "C" int fx_bias_act_f64(fx_ctx*, double*, const double*, int64_t, int64_t, int64_t, int);

namespace {
using namespace igemm;

int bias_act_t(fx_ctx* c, float* y, const float* b, i64 rows, i64 cols, int act) { return fx_bias_act_f32(c, y, b, rows, cols, 1, act); }
int bias_act_t(fx_ctx* c, double* y, const double* b, i64 rows, i64 cols, int act) { return fx_bias_act_f64(c, y, b, rows, cols, 1, act); }
// out[m] = sum over k of a[k][m] for a stored [K, M]
int col_sum_t(fx_ctx* c, const float* a, float* out, i64 K, i64 M) { return fx_bias_grad_f32(c, a, out, K, M, 1); }
int col_sum_t(fx_ctx* c, const double* a, double* out, i64 K, i64 M) { return fx_bias_grad_f64(c, a, out, K, M, 1); }
int relu_bwd_t(fx_ctx* c, const float* g, const float* x, float* o, i64 n) { return fx_relu_bwd_f32(c, g, x, o, n); }
int relu_bwd_t(fx_ctx* c, const double* g, const double* x, double* o, i64 n) { return fx_relu_bwd_f64(c, g, x, o, n); }

typedef Tile<128, 128, 16, 64, 64> TileBig;    // 4 waves, 64x64 each
typedef Tile<64, 64, 16, 32, 32> TileSmall;    // 4 waves, 32x32 each

template <typename T, class Cfg, bool TA, bool TB>
int run(fx_ctx* c, i64 M, i64 N, i64 K, const T* A, const T* B, T* C, const T* bias, int relu, bool* bias_pending) {
    // A stored [M,K] (k contiguous) unless TA ([K,M], m contiguous); B stored [K,N] (n contiguous) unless TB ([N,K]).
    MatLoader<T, !TA> al{A, TA ? M : K, (int)M};
    MatLoader<T, TB> bl{B, TB ? K : N, (int)N};
    const i64 tiles = fx::ceil_div(M, Cfg::BM) * fx::ceil_div(N, Cfg::BN);
    int kps = 0;
    const int splits = choose_splits(tiles, K, Cfg::BK, (i64)c->num_cus * 2, &kps);
    if (splits == 1) {
        if (bias) {  // bias (+ReLU) in the epilogue
            MatStore<T, true> ep{C, N, 0, (int)M, (int)N, bias, relu};
            return launch<T, Cfg>(c, al, bl, ep, M, N, K, 1, kps);
        }
        MatStore<T> ep{C, N, 0, (int)M, (int)N};
        return launch<T, Cfg>(c, al, bl, ep, M, N, K, 1, kps);
    }
    // split-K: the bias (and ReLU) ride in the ordered sum's store where its indices fit 32 bits, else the caller adds them after it
    const bool in_sum = bias != nullptr && M * N <= 0x7fffffff;
    *bias_pending = bias != nullptr && !in_sum;
    T* part = (T*)c->get_scratch((i64)splits * M * N * (i64)sizeof(T));
    if (!part) return FX_ERR_OOM;
    MatStore<T> ep{part, N, M * N, (int)M, (int)N};
    if (int rc = launch<T, Cfg>(c, al, bl, ep, M, N, K, splits, kps)) return rc;
    return launch_splitk_reduce<T>(c, part, C, M * N, splits, in_sum ? bias : nullptr, N, relu);
}

template <typename T, class Cfg>
int run_trans(fx_ctx* c, int ta, int tb, i64 M, i64 N, i64 K, const T* A, const T* B, T* C, const T* bias, int relu, bool* pend) {
    if (!ta && !tb) return run<T, Cfg, false, false>(c, M, N, K, A, B, C, bias, relu, pend);
    if (!ta && tb) return run<T, Cfg, false, true>(c, M, N, K, A, B, C, bias, relu, pend);
    if (ta && !tb) return run<T, Cfg, true, false>(c, M, N, K, A, B, C, bias, relu, pend);
    return run<T, Cfg, true, true>(c, M, N, K, A, B, C, bias, relu, pend);
}

// the one-launch small-product kernel; with K split over blocks, its partial results and their ordered sum (bias and ReLU in the sum's store)
int small_launch(fx_ctx* c, const gsmall::Plan& pl, bool ta, bool tb, i64 M, i64 N, i64 K, const float* A, const float* B, float* C, const float* bias,
                 int relu, float* part, float* asum) {
    return gsmall::run(c, pl, ta, tb, M, N, K, A, B, C, bias, relu, part, asum);
}
int small_launch(fx_ctx* c, const gsmall::Plan& pl, bool ta, bool tb, i64 M, i64 N, i64 K, const double* A, const double* B, double* C,
                 const double* bias, int relu, double* part, double* asum) {
    return gsmall::run_f64(c, pl, ta, tb, M, N, K, A, B, C, bias, relu, part, asum);
}
// asum (optional, only with an unsplit reduction): the row sums of op(A) from the same launch
template <typename T>
int small_product(fx_ctx* c, const gsmall::Plan& pl, bool ta, bool tb, i64 M, i64 N, i64 K, const T* A, const T* B, T* C, const T* bias, int relu,
                  T* asum = nullptr) {
    T* part = nullptr;
    if (pl.splits > 1) {
        part = (T*)c->get_scratch(gsmall::workspace_bytes<T>(pl, M, N));
        if (!part) return FX_ERR_OOM;
    }
    if (int rc = small_launch(c, pl, ta, tb, M, N, K, A, B, C, bias, relu, part, asum)) return rc;
    return pl.splits > 1 ? launch_splitk_reduce<T>(c, part, C, M * N, pl.splits, bias, N, relu) : FX_OK;
}

// asum_done (optional): with asum != null, set when the launch that computed C also wrote asum[m] = sum over k of op(A)[m][k]
template <typename T>
int gemm(fx_ctx* c, int ta, int tb, i64 M, i64 N, i64 K, const T* A, const T* B, T* C, const T* bias = nullptr, int relu = 0, T* asum = nullptr,
         bool* asum_done = nullptr) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(M >= 0 && N >= 0 && K >= 0, "fx_gemm: negative dimension");
    if (M == 0 || N == 0) return FX_OK;
    FX_REQUIRE(A && B && C, "fx_gemm: null pointer");
    FX_REQUIRE(M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31), "fx_gemm: dimension exceeds 2^31");
    // 32-bit byte offsets inside one 128-row tile of a k-contiguous operand
    FX_REQUIRE(K * 128 * (i64)sizeof(T) < (1ll << 32), "fx_gemm: K = %lld is too large for this build", (long long)K);
    bool pending = false;
    {
        std::lock_guard<std::mutex> lk(c->launch_mutex);
        int rc;
        bool lds_path = false;
        if constexpr (sizeof(T) == 4) {
            static const bool generic_only = std::getenv("FX_GEMM_GENERIC") != nullptr;  // A/B timing switch
            const glk::Plan pl = glk::make_plan(c->num_cus, ta != 0, tb != 0, M, N, K, ta ? M : K, tb ? K : N);
            lds_path = pl.ok && !generic_only && fx::aligned16(A) && fx::aligned16(B) && fx::aligned16(C);
            if (lds_path) rc = glk::run(c, pl, ta != 0, tb != 0, M, N, K, A, B, C, bias, relu);
            else if (!generic_only && gthin::eligible(c->num_cus, ta != 0, tb != 0, M, N, K)) {
                lds_path = true;
                rc = gthin::run(c, M, N, K, A, B, C, bias, relu, asum);
                if (asum) *asum_done = true;
            } else if (!generic_only) {
                const gsmall::Plan sp = gsmall::make_plan<float>(c->num_cus, ta != 0, tb != 0, M, N, K, A, B, asum == nullptr);
                if (sp.ok) {
                    lds_path = true;
                    const bool with_sum = asum != nullptr && sp.splits == 1;
                    rc = small_product<float>(c, sp, ta != 0, tb != 0, M, N, K, A, B, C, bias, relu, with_sum ? asum : nullptr);
                    if (with_sum) *asum_done = true;
                }
            }
        }
        if constexpr (sizeof(T) == 8) {
            static const bool generic_only = std::getenv("FX_GEMM_GENERIC") != nullptr;
            if (!generic_only) {
                const gsmall::Plan sp = gsmall::make_plan<double>(c->num_cus, ta != 0, tb != 0, M, N, K, A, B);
                if (sp.ok) {
                    lds_path = true;
                    const bool with_sum = asum != nullptr && sp.splits == 1;
                    rc = small_product<double>(c, sp, ta != 0, tb != 0, M, N, K, A, B, C, bias, relu, with_sum ? asum : nullptr);
                    if (with_sum) *asum_done = true;
                }
            }
        }
        if (lds_path) {
        } else if (K == 0) {  // empty sum
            rc = launch_zero<T>(c, C, M * N);
            pending = bias != nullptr;
        } else if (M >= 128 && N >= 128) rc = run_trans<T, TileBig>(c, ta, tb, M, N, K, A, B, C, bias, relu, &pending);
        else rc = run_trans<T, TileSmall>(c, ta, tb, M, N, K, A, B, C, bias, relu, &pending);
        if (rc) return rc;
    }
    return pending ? bias_act_t(c, C, bias, M, N, relu) : FX_OK;
}
}  // namespace

// C[M,N] = A^T . B for A stored [K, M] and B stored [K, N], plus colsum[m] = sum over k of A[k][m]: the weight and the bias
// gradient of a Linear layer from its upstream gradient A = dY [batch, out] and its input B = X [batch, in].  Small and thin
// products compute the sums in the product's launch; the others run the bias-gradient kernel after it.
template <typename T>
int gemm_tn_colsum(fx_ctx* c, i64 M, i64 N, i64 K, const T* A, const T* B, T* C, T* colsum) {
    FX_REQUIRE(colsum != nullptr, "fx_gemm_tn_colsum: null pointer");
    FX_REQUIRE(M >= 1 && N >= 1 && K >= 1, "fx_gemm_tn_colsum: empty dimension");
    bool done = false;
    if (int rc = gemm<T>(c, 1, 0, M, N, K, A, B, C, nullptr, 0, colsum, &done)) return rc;
    return done ? FX_OK : col_sum_t(c, A, colsum, K, M);
}
// Linear's backward products in one call: dX[B, in] = dY[B, out] . W[out, in], dW[out, in] = dY^T . X[B, in] and (optionally)
// db[out] = the column sums of dY.  Where both products are small ones (each would run the one-launch small-product kernel on its
// own) they share a launch; the results have the bits of the separate calls either way.
// relu_below: X is the output of a ReLU, and dX comes out as the gradient of that ReLU's input, (dY . W) * (X > 0 ? 1 : 0) --
// fx_relu_bwd's operation, in the store of the product where the two share a launch, as a pass over dX otherwise.
template <typename T>
int linear_bwd(fx_ctx* c, i64 Bn, i64 I, i64 O, const T* g, const T* W, const T* X, T* dX, T* dW, T* db, int relu_below) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(g && W && X && dX && dW, "fx_linear_bwd: null pointer");
    FX_REQUIRE(Bn >= 1 && I >= 1 && O >= 1 && Bn < (1ll << 31) && I < (1ll << 31) && O < (1ll << 31), "fx_linear_bwd: bad dimensions");
    static const bool generic_only = std::getenv("FX_GEMM_GENERIC") != nullptr;
    if (!generic_only) {
        bool other = false;  // a product that gemm() would give to the slab or the thin kernel
        if constexpr (sizeof(T) == 4) {
            other = glk::make_plan(c->num_cus, false, false, Bn, I, O, O, I).ok || glk::make_plan(c->num_cus, true, false, O, I, Bn, O, I).ok ||
                    gthin::eligible(c->num_cus, false, false, Bn, I, O) || gthin::eligible(c->num_cus, true, false, O, I, Bn);
        }
        if (!other) {
            const gsmall::Plan p0 = gsmall::make_plan<T>(c->num_cus, false, false, Bn, I, O, g, W);
            const gsmall::Plan p1 = gsmall::make_plan<T>(c->num_cus, true, false, O, I, Bn, g, X);
            if (p0.ok && p1.ok && p0.splits == 1 && p1.splits == 1) {
                std::lock_guard<std::mutex> lk(c->launch_mutex);
                return gsmall::run_pair(c, p0, p1, Bn, I, O, g, W, dX, O, I, Bn, g, X, dW, db, relu_below ? X : nullptr);
            }
        }
    }
    if (int rc = gemm<T>(c, 0, 0, Bn, I, O, g, W, dX)) return rc;
    if (relu_below) {
        if (int rc = relu_bwd_t(c, dX, X, dX, Bn * I)) return rc;
    }
    return db ? gemm_tn_colsum<T>(c, O, I, Bn, g, X, dW, db) : gemm<T>(c, 1, 0, O, I, Bn, g, X, dW);
}
extern "C" int fx_linear_bwd_f32(fx_ctx* c, int64_t B, int64_t in, int64_t out, const float* dY, const float* W, const float* X, float* dX,
                                 float* dW, float* db, int relu_below) {
    return linear_bwd<float>(c, B, in, out, dY, W, X, dX, dW, db, relu_below);
}
extern "C" int fx_linear_bwd_f64(fx_ctx* c, int64_t B, int64_t in, int64_t out, const double* dY, const double* W, const double* X, double* dX,
                                 double* dW, double* db, int relu_below) {
    return linear_bwd<double>(c, B, in, out, dY, W, X, dX, dW, db, relu_below);
}
extern "C" int fx_gemm_tn_colsum_f32(fx_ctx* c, int64_t M, int64_t N, int64_t K, const float* A, const float* B, float* C, float* colsum) {
    return gemm_tn_colsum<float>(c, M, N, K, A, B, C, colsum);
}
extern "C" int fx_gemm_tn_colsum_f64(fx_ctx* c, int64_t M, int64_t N, int64_t K, const double* A, const double* B, double* C, double* colsum) {
    return gemm_tn_colsum<double>(c, M, N, K, A, B, C, colsum);
}
extern "C" int fx_gemm_f32(fx_ctx* c, int ta, int tb, int64_t M, int64_t N, int64_t K, const float* A, const float* B, float* C) {
    return gemm<float>(c, ta, tb, M, N, K, A, B, C);
}
extern "C" int fx_gemm_f64(fx_ctx* c, int ta, int tb, int64_t M, int64_t N, int64_t K, const double* A, const double* B, double* C) {
    return gemm<double>(c, ta, tb, M, N, K, A, B, C);
}
// C = act(op(A).op(B) + bias[n]): the bias add (and ReLU) ride in the GEMM's store unless the product was split along K.
extern "C" int fx_gemm_bias_act_f32(fx_ctx* c, int ta, int tb, int64_t M, int64_t N, int64_t K, const float* A, const float* B,
                                    const float* bias, float* C, int act) {
    FX_REQUIRE(bias != nullptr, "fx_gemm_bias_act: null bias");
    FX_REQUIRE(act == 0 || act == 1, "fx_gemm_bias_act: act must be 0 (none) or 1 (relu)");
    return gemm<float>(c, ta, tb, M, N, K, A, B, C, bias, act);
}
extern "C" int fx_gemm_bias_act_f64(fx_ctx* c, int ta, int tb, int64_t M, int64_t N, int64_t K, const double* A, const double* B,
                                    const double* bias, double* C, int act) {
    FX_REQUIRE(bias != nullptr, "fx_gemm_bias_act: null bias");
    FX_REQUIRE(act == 0 || act == 1, "fx_gemm_bias_act: act must be 0 (none) or 1 (relu)");
    return gemm<double>(c, ta, tb, M, N, K, A, B, C, bias, act);
}
