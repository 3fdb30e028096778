// Batch normalisation over the channel axis of a contiguous [outer, C, inner] view ([N, C, H, W]: outer = N,
// inner = H*W; [N, F]: outer = N, C = F, inner = 1).  The reference composes it from graph operators
// (src/nn/layers/norm.rs:192-336): Mean -> BroadcastTo -> Sub -> Mul -> Mean -> BroadcastTo -> AddScalar -> Sqrt -> Div
// -> Mul -> Add, about 15 full-size passes forward and twice that backward.  Here:
//   stats   one read of x: per-channel mean and biased variance (+ the running-statistics update, norm.rs:127-164)
//   fwd     y = ((x - mean) / sqrt(var + eps)) * gamma + beta, the composed operations in the composed order
//           (this file is built without a*b+c contraction), so y equals the composed path bit for bit given mean/var
//   bwd     two reads of (dy, x): channel sums, then dx = (gamma/std) * (dy - mean(dy) - xc * mean(dy*xc)/std^2)
//   A ReLU that follows the layer can ride along: fwd applies it in the store, bwd masks dy where the activation is 0.
// All three are HBM-bound: sizeof(T) * n * {1, 2, 5} bytes.
//
// Moments are combined with the pairwise update of Chan, Golub & LeVeque (count, mean, M2): every thread folds
// register groups (exact two-pass inside a group) into its running triple, threads merge in a fixed tree, slices in
// slice order.  No atomics; results depend only on the shape.
#include <algorithm>

#include "common.hpp"

namespace {

template <typename T> __device__ __forceinline__ T dev_sqrt(T x);
template <> __device__ __forceinline__ float dev_sqrt<float>(float x) { return sqrtf(x); }
template <> __device__ __forceinline__ double dev_sqrt<double>(double x) { return sqrt(x); }
__device__ __forceinline__ float dev_fma(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ __forceinline__ double dev_fma(double a, double b, double c) { return __builtin_fma(a, b, c); }
__device__ __forceinline__ float dev_rcp(float x) { return __builtin_amdgcn_rcpf(x); }
__device__ __forceinline__ double dev_rcp(double x) { return 1.0 / x; }

template <typename T> struct Moments {
    T n, mean, m2;
    __device__ __forceinline__ void init() { n = T(0); mean = T(0); m2 = T(0); }
    // fold in another set of nb > 0 samples with mean mb and centred sum of squares m2b
    __device__ __forceinline__ void merge(T nb, T mb, T m2b) {
        const T nn = n + nb;
        const T f = nb * dev_rcp(nn);
        const T d = mb - mean;
        mean = dev_fma(d, f, mean);
        m2 = m2 + dev_fma(d * d, n * f, m2b);
        n = nn;
    }
    __device__ __forceinline__ void merge_any(T nb, T mb, T m2b) { if (nb > T(0)) merge(nb, mb, m2b); }
    // K register values: exact two-pass moments of the group, then one merge
    template <int K> __device__ __forceinline__ void take(const T (&x)[K]) {
        T s = x[0];
#pragma unroll
        for (int k = 1; k < K; ++k) s = s + x[k];
        const T m = s * T(1.0 / K);
        T q = T(0);
#pragma unroll
        for (int k = 0; k < K; ++k) { const T d = x[k] - m; q = dev_fma(d, d, q); }
        merge(T(K), m, q);
    }
};

// block-wide merge of per-thread moments in a fixed tree; result in thread 0
template <typename T> __device__ __forceinline__ void block_merge(Moments<T>& a, T (*sm)[256]) {
    sm[0][threadIdx.x] = a.n; sm[1][threadIdx.x] = a.mean; sm[2][threadIdx.x] = a.m2;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) {
        if ((int)threadIdx.x < w) {
            a.merge_any(sm[0][threadIdx.x + w], sm[1][threadIdx.x + w], sm[2][threadIdx.x + w]);
            sm[0][threadIdx.x] = a.n; sm[1][threadIdx.x] = a.mean; sm[2][threadIdx.x] = a.m2;
        }
        __syncthreads();
    }
}

// Walks the (row, vector) pairs of rows [o0, o1) of channel c: pair q -> row o0 + q / nv, vector q % nv; thread t
// takes q = t, t + 256, ...  F(ptr) is called with the address of each vector, four independent loads per trip.
// (dq, dr) = (256 / nv, 256 % nv) steps the pair without a division per load.
struct PairWalk {
    i64 o, iv;
    i64 dq, dr, nv;
    __device__ __forceinline__ PairWalk(i64 o0, i64 nv_, int t) : nv(nv_) {
        o = o0 + t / nv_; iv = t % nv_;
        dq = 256 / nv_; dr = 256 % nv_;
    }
    __device__ __forceinline__ void step() {
        o += dq; iv += dr;
        if (iv >= nv) { iv -= nv; ++o; }
    }
};

// ---- statistics, planar form: grid (C, slices); partial triple of (slice, c) at part[(slice*C + c)*3] --------------
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void bn_stats_planar_kernel(const T* __restrict__ x, T* __restrict__ part, i64 outer, i64 C,
                                                              i64 inner, i64 rows_per_slice) {
    constexpr int V = VEC ? 16 / (int)sizeof(T) : 1;
    typedef T vec_t __attribute__((ext_vector_type(V)));
    __shared__ T sm[3][256];
    const i64 c = blockIdx.x, slice = blockIdx.y;
    const i64 o0 = slice * rows_per_slice, o1 = min(outer, o0 + rows_per_slice);
    const i64 nv = inner / V, pairs = (o1 - o0) * nv;
    Moments<T> acc;
    acc.init();
    PairWalk w(o0, nv, (int)threadIdx.x);
    i64 q = threadIdx.x;
    for (; q + 3 * 256 < pairs; q += 4 * 256) {
        vec_t v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            v[u] = *reinterpret_cast<const vec_t*>(x + (w.o * C + c) * inner + w.iv * V);
            w.step();
        }
        T g[4 * V];
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int e = 0; e < V; ++e) g[u * V + e] = v[u][e];
        acc.template take<4 * V>(g);
    }
    for (; q < pairs; q += 256) {
        const vec_t v = *reinterpret_cast<const vec_t*>(x + (w.o * C + c) * inner + w.iv * V);
        w.step();
        T g[V];
#pragma unroll
        for (int e = 0; e < V; ++e) g[e] = v[e];
        acc.template take<V>(g);
    }
    block_merge<T>(acc, sm);
    if (threadIdx.x == 0) {
        T* p = part + (slice * C + c) * 3;
        p[0] = acc.n; p[1] = acc.mean; p[2] = acc.m2;
    }
}

// ---- statistics, column form (short inner): x viewed as [outer, Q = C*inner]; thread per column, rows of the slice in
// groups of eight; partial triple of (slice, column) at part[(slice*Q + column)*3] ------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void bn_stats_column_kernel(const T* __restrict__ x, T* __restrict__ part, i64 outer, i64 Q,
                                                              i64 rows_per_slice) {
    const i64 col = (i64)blockIdx.x * 256 + threadIdx.x, slice = blockIdx.y;
    if (col >= Q) return;
    const i64 o0 = slice * rows_per_slice, o1 = min(outer, o0 + rows_per_slice);
    Moments<T> acc;
    acc.init();
    i64 o = o0;
    for (; o + 8 <= o1; o += 8) {
        T g[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) g[u] = x[(o + u) * Q + col];
        acc.template take<8>(g);
    }
    for (; o < o1; ++o) {
        T g[1] = {x[o * Q + col]};
        acc.template take<1>(g);
    }
    T* p = part + (slice * Q + col) * 3;
    p[0] = acc.n; p[1] = acc.mean; p[2] = acc.m2;
}

// one wave per channel: lane l folds partial triples l, l + 64, ... (in (slice, column) order), then the lanes merge in a
// fixed shuffle tree
template <typename T>
__global__ __launch_bounds__(64) void bn_stats_final_kernel(const T* __restrict__ part, T* __restrict__ mean, T* __restrict__ var,
                                                            T* __restrict__ run_mean, T* __restrict__ run_var, T mom, T one_minus_mom,
                                                            i64 C, i64 per_channel, int slices) {
    const i64 c = blockIdx.x;
    const i64 count = (i64)slices * per_channel;
    Moments<T> acc;
    acc.init();
    for (i64 k = threadIdx.x; k < count; k += 64) {
        const i64 z = k / per_channel, j = k - z * per_channel;
        const T* p = part + ((z * C + c) * per_channel + j) * 3;
        acc.merge_any(p[0], p[1], p[2]);
    }
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) {
        const T on = __shfl_down(acc.n, d, 64), om = __shfl_down(acc.mean, d, 64), o2 = __shfl_down(acc.m2, d, 64);
        if ((int)threadIdx.x + d < 64) acc.merge_any(on, om, o2);
    }
    if (threadIdx.x != 0) return;
    const T m = acc.mean, v = acc.m2 / acc.n;
    mean[c] = m;
    var[c] = v;
    // running = running * (1 - momentum) + batch * momentum, norm.rs:144-161 (biased variance, as the reference keeps it)
    if (run_mean) run_mean[c] = run_mean[c] * one_minus_mom + m * mom;
    if (run_var) run_var[c] = run_var[c] * one_minus_mom + v * mom;
}

struct Split {
    i64 slices, rows_per_slice;
};
// enough blocks to fill the chip, at least ~16k elements per block
inline Split split_rows(const fx_ctx* c, i64 outer, i64 columns_of_blocks, i64 elems_per_row_per_block) {
    i64 slices = std::max<i64>(1, std::min<i64>((i64)c->num_cus * 4 / std::max<i64>(1, columns_of_blocks), 65535));
    const i64 min_rows = std::max<i64>(1, 16384 / std::max<i64>(1, elems_per_row_per_block));
    slices = std::max<i64>(1, std::min<i64>(slices, outer / min_rows));
    const i64 rps = fx::ceil_div(outer, slices);
    return Split{fx::ceil_div(outer, rps), rps};
}

template <typename T>
int bn_stats(fx_ctx* c, const T* x, T* mean, T* var, T* run_mean, T* run_var, double momentum, i64 outer, i64 C, i64 inner) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(outer >= 1 && C >= 1 && inner >= 1, "fx_batchnorm_stats: bad view [%lld, %lld, %lld]", (long long)outer, (long long)C,
               (long long)inner);
    FX_REQUIRE(x && mean && var, "fx_batchnorm_stats: null pointer");
    // Sample counts travel in T: a thread's own count stays far below 2^24 (it grows by whole register groups and a
    // block has 256 threads), the merged counts above that are only weights of the pairwise merge (relative error 6e-8).
    FX_REQUIRE(C <= 0x7fffffff && inner <= 0x7fffffff && outer * inner < (1ll << 31) * (sizeof(T) == 4 ? 1 : (1ll << 17)),
               "fx_batchnorm_stats: view too large");
    constexpr int V = 16 / (int)sizeof(T);
    std::lock_guard<std::mutex> lk(c->launch_mutex);
    i64 per_channel;
    Split sp;
    T* part;
    if (inner >= 16) {
        sp = split_rows(c, outer, C, inner);
        per_channel = 1;
        part = (T*)c->get_scratch(sp.slices * C * 3 * (i64)sizeof(T));
        if (!part) return FX_ERR_OOM;
        const dim3 grid((unsigned)C, (unsigned)sp.slices);
        if (inner % V == 0 && fx::aligned16(x)) bn_stats_planar_kernel<T, true><<<grid, dim3(256), 0, c->stream>>>(x, part, outer, C, inner, sp.rows_per_slice);
        else bn_stats_planar_kernel<T, false><<<grid, dim3(256), 0, c->stream>>>(x, part, outer, C, inner, sp.rows_per_slice);
    } else {
        const i64 Q = C * inner, col_blocks = fx::ceil_div(Q, 256);
        FX_REQUIRE(col_blocks <= 0x7fffffff, "fx_batchnorm_stats: too many channels");
        sp = split_rows(c, outer, col_blocks, 256);
        per_channel = inner;
        part = (T*)c->get_scratch(sp.slices * Q * 3 * (i64)sizeof(T));
        if (!part) return FX_ERR_OOM;
        bn_stats_column_kernel<T><<<dim3((unsigned)col_blocks, (unsigned)sp.slices), dim3(256), 0, c->stream>>>(x, part, outer, Q, sp.rows_per_slice);
    }
    FX_LAUNCH_CHECK();
    bn_stats_final_kernel<T><<<dim3((unsigned)C), dim3(64), 0, c->stream>>>(
        part, mean, var, run_mean, run_var, (T)momentum, (T)(1.0 - momentum), C, per_channel, (int)sp.slices);
    FX_LAUNCH_CHECK();
    return FX_OK;
}

// ---- forward: y = ((x - mean) / sqrt(var + eps)) * gamma + beta ------------------------------------------------------
template <typename T, bool VEC, bool RELU>
__global__ __launch_bounds__(256) void bn_fwd_kernel(const T* __restrict__ x, const T* __restrict__ mean, const T* __restrict__ var,
                                                     const T* __restrict__ gamma, const T* __restrict__ beta, T eps, T* __restrict__ y,
                                                     i64 n, uint32_t C, uint32_t inner) {
    constexpr int V = VEC ? 16 / (int)sizeof(T) : 1;
    typedef T vec_t __attribute__((ext_vector_type(V)));
    const i64 i = ((i64)blockIdx.x * 256 + threadIdx.x) * V;
    if (i >= n) return;
    const uint32_t c = (uint32_t)((i / inner) % C);
    const T m = mean[c], sd = dev_sqrt<T>(var[c] + eps), g = gamma[c], b = beta[c];
    vec_t v = *reinterpret_cast<const vec_t*>(x + i);
#pragma unroll
    for (int u = 0; u < V; ++u) {
        T r = ((v[u] - m) / sd) * g + b;
        if (RELU) r = r > T(0) ? r : T(0);  // ReLU as the forward kernel does it: x > 0 ? x : 0
        v[u] = r;
    }
    *reinterpret_cast<vec_t*>(y + i) = v;
}

template <typename T>
int bn_fwd(fx_ctx* c, const T* x, const T* mean, const T* var, const T* gamma, const T* beta, double eps, T* y, i64 outer, i64 C,
           i64 inner, int act) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(outer >= 0 && C >= 1 && inner >= 1, "fx_batchnorm_fwd: bad view");
    FX_REQUIRE(act == 0 || act == 1, "fx_batchnorm_fwd: act must be 0 (none) or 1 (relu)");
    const i64 n = outer * C * inner;
    if (n == 0) return FX_OK;
    FX_REQUIRE(x && mean && var && gamma && beta && y, "fx_batchnorm_fwd: null pointer");
    FX_REQUIRE(C <= 0x7fffffff && inner <= 0x7fffffff, "fx_batchnorm_fwd: view too large");
    constexpr int V = 16 / (int)sizeof(T);
    const bool vec = inner % V == 0 && fx::aligned16(x) && fx::aligned16(y);
    const i64 blocks = fx::ceil_div(vec ? n / V : n, 256);
    FX_REQUIRE(blocks <= 0x7fffffff, "fx_batchnorm_fwd: too many elements");
    const dim3 grid((unsigned)blocks), blk(256);
    const T e = (T)eps;
    const uint32_t Cu = (uint32_t)C, iu = (uint32_t)inner;
    if (vec && act) bn_fwd_kernel<T, true, true><<<grid, blk, 0, c->stream>>>(x, mean, var, gamma, beta, e, y, n, Cu, iu);
    else if (vec) bn_fwd_kernel<T, true, false><<<grid, blk, 0, c->stream>>>(x, mean, var, gamma, beta, e, y, n, Cu, iu);
    else if (act) bn_fwd_kernel<T, false, true><<<grid, blk, 0, c->stream>>>(x, mean, var, gamma, beta, e, y, n, Cu, iu);
    else bn_fwd_kernel<T, false, false><<<grid, blk, 0, c->stream>>>(x, mean, var, gamma, beta, e, y, n, Cu, iu);
    FX_LAUNCH_CHECK();
    return FX_OK;
}

// ---- backward, stage 1: per (slice, column) sums of dy and dy * (x - mean) -------------------------------------------
// MASK: dy is the gradient of relu(y); yact holds relu(y) and dy counts only where yact > 0 (ReLU::gradient, unary.rs:358-375).
template <typename T, bool VEC, bool MASK>
__global__ __launch_bounds__(256) void bn_bwd_sums_planar_kernel(const T* __restrict__ dy, const T* __restrict__ x,
                                                                 const T* __restrict__ yact, const T* __restrict__ mean,
                                                                 T* __restrict__ part, i64 outer, i64 C, i64 inner, i64 rows_per_slice) {
    constexpr int V = VEC ? 16 / (int)sizeof(T) : 1;
    typedef T vec_t __attribute__((ext_vector_type(V)));
    __shared__ T sm[2][256];
    const i64 c = blockIdx.x, slice = blockIdx.y;
    const i64 o0 = slice * rows_per_slice, o1 = min(outer, o0 + rows_per_slice);
    const i64 nv = inner / V, pairs = (o1 - o0) * nv;
    const T m = mean[c];
    vec_t s1 = vec_t(T(0)), s2 = vec_t(T(0));
    PairWalk w(o0, nv, (int)threadIdx.x);
    i64 q = threadIdx.x;
    for (; q + 3 * 256 < pairs; q += 4 * 256) {
        vec_t g[4], v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const i64 off = (w.o * C + c) * inner + w.iv * V;
            g[u] = *reinterpret_cast<const vec_t*>(dy + off);
            v[u] = *reinterpret_cast<const vec_t*>(x + off);
            if (MASK) {
                const vec_t a = *reinterpret_cast<const vec_t*>(yact + off);
#pragma unroll
                for (int e = 0; e < V; ++e) g[u][e] = a[e] > T(0) ? g[u][e] : T(0);
            }
            w.step();
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            s1 = s1 + g[u];
#pragma unroll
            for (int e = 0; e < V; ++e) s2[e] = dev_fma(g[u][e], v[u][e] - m, s2[e]);
        }
    }
    for (; q < pairs; q += 256) {
        const i64 off = (w.o * C + c) * inner + w.iv * V;
        vec_t g = *reinterpret_cast<const vec_t*>(dy + off);
        const vec_t v = *reinterpret_cast<const vec_t*>(x + off);
        if (MASK) {
            const vec_t a = *reinterpret_cast<const vec_t*>(yact + off);
#pragma unroll
            for (int e = 0; e < V; ++e) g[e] = a[e] > T(0) ? g[e] : T(0);
        }
        w.step();
        s1 = s1 + g;
#pragma unroll
        for (int e = 0; e < V; ++e) s2[e] = dev_fma(g[e], v[e] - m, s2[e]);
    }
    T a = T(0), b = T(0);
#pragma unroll
    for (int e = 0; e < V; ++e) { a = a + s1[e]; b = b + s2[e]; }
    sm[0][threadIdx.x] = a; sm[1][threadIdx.x] = b;
    __syncthreads();
    for (int h = 128; h > 0; h >>= 1) {
        if ((int)threadIdx.x < h) {
            sm[0][threadIdx.x] = sm[0][threadIdx.x] + sm[0][threadIdx.x + h];
            sm[1][threadIdx.x] = sm[1][threadIdx.x] + sm[1][threadIdx.x + h];
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        T* p = part + (slice * C + c) * 2;
        p[0] = sm[0][0]; p[1] = sm[1][0];
    }
}

template <typename T>
__global__ __launch_bounds__(256) void bn_bwd_sums_column_kernel(const T* __restrict__ dy, const T* __restrict__ x,
                                                                 const T* __restrict__ yact, const T* __restrict__ mean,
                                                                 T* __restrict__ part, i64 outer, i64 Q, uint32_t inner, i64 rows_per_slice) {
    const i64 col = (i64)blockIdx.x * 256 + threadIdx.x, slice = blockIdx.y;
    if (col >= Q) return;
    const i64 o0 = slice * rows_per_slice, o1 = min(outer, o0 + rows_per_slice);
    const T m = mean[col / inner];
    T a = T(0), b = T(0);
    for (i64 o = o0; o < o1; ++o) {
        T g = dy[o * Q + col];
        if (yact) g = yact[o * Q + col] > T(0) ? g : T(0);
        a = a + g;
        b = dev_fma(g, x[o * Q + col] - m, b);
    }
    T* p = part + (slice * Q + col) * 2;
    p[0] = a; p[1] = b;
}

// one wave per channel: dbeta, dgamma and the coefficients of the dx kernel (coef[0..C) = gamma/std,
// coef[C..2C) = mean(dy), coef[2C..3C) = mean(dy*xc)/std^2); partials summed lane-strided, then a fixed shuffle tree
template <typename T>
__global__ __launch_bounds__(64) void bn_bwd_final_kernel(const T* __restrict__ part, const T* __restrict__ var,
                                                          const T* __restrict__ gamma, T eps, T* __restrict__ dgamma,
                                                          T* __restrict__ dbeta, T* __restrict__ coef, T count, i64 C, i64 per_channel,
                                                          int slices) {
    const i64 c = blockIdx.x;
    const i64 np = (i64)slices * per_channel;
    T a = T(0), b = T(0);
    for (i64 k = threadIdx.x; k < np; k += 64) {
        const i64 z = k / per_channel, j = k - z * per_channel;
        const T* p = part + ((z * C + c) * per_channel + j) * 2;
        a = a + p[0];
        b = b + p[1];
    }
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) {
        const T oa = __shfl_down(a, d, 64), ob = __shfl_down(b, d, 64);
        if ((int)threadIdx.x + d < 64) { a = a + oa; b = b + ob; }
    }
    if (threadIdx.x != 0) return;
    const T sd = dev_sqrt<T>(var[c] + eps);
    dbeta[c] = a;
    dgamma[c] = b / sd;
    coef[c] = gamma[c] / sd;
    coef[C + c] = a / count;
    coef[2 * C + c] = (b / count) / (sd * sd);
}

// stage 2, batch statistics: dx = (dy - k1 - (x - mean) * k2) * (gamma/std)
template <typename T, bool VEC, bool MASK>
__global__ __launch_bounds__(256) void bn_bwd_dx_kernel(const T* __restrict__ dy, const T* __restrict__ x, const T* __restrict__ yact,
                                                        const T* __restrict__ mean, const T* __restrict__ coef, T* __restrict__ dx, i64 n,
                                                        uint32_t C, uint32_t inner) {
    constexpr int V = VEC ? 16 / (int)sizeof(T) : 1;
    typedef T vec_t __attribute__((ext_vector_type(V)));
    const i64 i = ((i64)blockIdx.x * 256 + threadIdx.x) * V;
    if (i >= n) return;
    const uint32_t c = (uint32_t)((i / inner) % C);
    const T m = mean[c], a = coef[c], k1 = coef[C + c], k2 = coef[2 * C + c];
    vec_t g = *reinterpret_cast<const vec_t*>(dy + i);
    const vec_t v = *reinterpret_cast<const vec_t*>(x + i);
    if (MASK) {
        const vec_t ya = *reinterpret_cast<const vec_t*>(yact + i);
#pragma unroll
        for (int u = 0; u < V; ++u) g[u] = ya[u] > T(0) ? g[u] : T(0);
    }
    vec_t r;
#pragma unroll
    for (int u = 0; u < V; ++u) r[u] = ((g[u] - k1) - (v[u] - m) * k2) * a;
    *reinterpret_cast<vec_t*>(dx + i) = r;
}

// stage 2, fixed (running) statistics: dx = (dy * gamma) / std, the composed Mul and Div gradients in their order
template <typename T, bool VEC, bool MASK>
__global__ __launch_bounds__(256) void bn_bwd_dx_fixed_kernel(const T* __restrict__ dy, const T* __restrict__ yact,
                                                              const T* __restrict__ var, const T* __restrict__ gamma, T eps,
                                                              T* __restrict__ dx, i64 n, uint32_t C, uint32_t inner) {
    constexpr int V = VEC ? 16 / (int)sizeof(T) : 1;
    typedef T vec_t __attribute__((ext_vector_type(V)));
    const i64 i = ((i64)blockIdx.x * 256 + threadIdx.x) * V;
    if (i >= n) return;
    const uint32_t c = (uint32_t)((i / inner) % C);
    const T sd = dev_sqrt<T>(var[c] + eps), gm = gamma[c];
    vec_t g = *reinterpret_cast<const vec_t*>(dy + i);
    if (MASK) {
        const vec_t ya = *reinterpret_cast<const vec_t*>(yact + i);
#pragma unroll
        for (int u = 0; u < V; ++u) g[u] = ya[u] > T(0) ? g[u] : T(0);
    }
#pragma unroll
    for (int u = 0; u < V; ++u) g[u] = (g[u] * gm) / sd;
    *reinterpret_cast<vec_t*>(dx + i) = g;
}

template <typename T>
int bn_bwd(fx_ctx* c, const T* dy, const T* x, const T* yact, const T* mean, const T* var, const T* gamma, double eps, T* dx, T* dgamma,
           T* dbeta, i64 outer, i64 C, i64 inner, int batch_stats) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(outer >= 1 && C >= 1 && inner >= 1, "fx_batchnorm_bwd: bad view");
    FX_REQUIRE(dy && x && mean && var && gamma && dgamma && dbeta, "fx_batchnorm_bwd: null pointer");
    FX_REQUIRE(C <= 0x7fffffff && inner <= 0x7fffffff, "fx_batchnorm_bwd: view too large");
    FX_REQUIRE(batch_stats == 0 || batch_stats == 1, "fx_batchnorm_bwd: batch_stats must be 0 or 1");
    constexpr int V = 16 / (int)sizeof(T);
    const i64 n = outer * C * inner;
    std::lock_guard<std::mutex> lk(c->launch_mutex);
    i64 per_channel, n_part;
    Split sp;
    const bool planar = inner >= 16;
    const i64 Q = C * inner, col_blocks = fx::ceil_div(Q, 256);
    if (planar) {
        sp = split_rows(c, outer, C, inner);
        per_channel = 1;
        n_part = sp.slices * C * 2;
    } else {
        FX_REQUIRE(col_blocks <= 0x7fffffff, "fx_batchnorm_bwd: too many channels");
        sp = split_rows(c, outer, col_blocks, 256);
        per_channel = inner;
        n_part = sp.slices * Q * 2;
    }
    const i64 coef_off = ((n_part * (i64)sizeof(T) + 255) / 256) * 256;
    char* sc = (char*)c->get_scratch(coef_off + 3 * C * (i64)sizeof(T));
    if (!sc) return FX_ERR_OOM;
    T* part = (T*)sc;
    T* coef = (T*)(sc + coef_off);
    if (planar) {
        const dim3 grid((unsigned)C, (unsigned)sp.slices);
        const bool v16 = inner % V == 0 && fx::aligned16(x) && fx::aligned16(dy) && (!yact || fx::aligned16(yact));
        const i64 rps = sp.rows_per_slice;
        if (v16 && yact) bn_bwd_sums_planar_kernel<T, true, true><<<grid, dim3(256), 0, c->stream>>>(dy, x, yact, mean, part, outer, C, inner, rps);
        else if (v16) bn_bwd_sums_planar_kernel<T, true, false><<<grid, dim3(256), 0, c->stream>>>(dy, x, yact, mean, part, outer, C, inner, rps);
        else if (yact) bn_bwd_sums_planar_kernel<T, false, true><<<grid, dim3(256), 0, c->stream>>>(dy, x, yact, mean, part, outer, C, inner, rps);
        else bn_bwd_sums_planar_kernel<T, false, false><<<grid, dim3(256), 0, c->stream>>>(dy, x, yact, mean, part, outer, C, inner, rps);
    } else {
        bn_bwd_sums_column_kernel<T><<<dim3((unsigned)col_blocks, (unsigned)sp.slices), dim3(256), 0, c->stream>>>(
            dy, x, yact, mean, part, outer, Q, (uint32_t)inner, sp.rows_per_slice);
    }
    FX_LAUNCH_CHECK();
    bn_bwd_final_kernel<T><<<dim3((unsigned)C), dim3(64), 0, c->stream>>>(
        part, var, gamma, (T)eps, dgamma, dbeta, coef, (T)(outer * inner), C, per_channel, (int)sp.slices);
    FX_LAUNCH_CHECK();
    if (!dx) return FX_OK;
    const bool vec = inner % V == 0 && fx::aligned16(x) && fx::aligned16(dy) && fx::aligned16(dx) && (!yact || fx::aligned16(yact));
    const i64 blocks = fx::ceil_div(vec ? n / V : n, 256);
    FX_REQUIRE(blocks <= 0x7fffffff, "fx_batchnorm_bwd: too many elements");
    const dim3 grid((unsigned)blocks), blk(256);
    const uint32_t Cu = (uint32_t)C, iu = (uint32_t)inner;
    if (batch_stats) {
        if (vec && yact) bn_bwd_dx_kernel<T, true, true><<<grid, blk, 0, c->stream>>>(dy, x, yact, mean, coef, dx, n, Cu, iu);
        else if (vec) bn_bwd_dx_kernel<T, true, false><<<grid, blk, 0, c->stream>>>(dy, x, yact, mean, coef, dx, n, Cu, iu);
        else if (yact) bn_bwd_dx_kernel<T, false, true><<<grid, blk, 0, c->stream>>>(dy, x, yact, mean, coef, dx, n, Cu, iu);
        else bn_bwd_dx_kernel<T, false, false><<<grid, blk, 0, c->stream>>>(dy, x, yact, mean, coef, dx, n, Cu, iu);
    } else {
        if (vec && yact) bn_bwd_dx_fixed_kernel<T, true, true><<<grid, blk, 0, c->stream>>>(dy, yact, var, gamma, (T)eps, dx, n, Cu, iu);
        else if (vec) bn_bwd_dx_fixed_kernel<T, true, false><<<grid, blk, 0, c->stream>>>(dy, yact, var, gamma, (T)eps, dx, n, Cu, iu);
        else if (yact) bn_bwd_dx_fixed_kernel<T, false, true><<<grid, blk, 0, c->stream>>>(dy, yact, var, gamma, (T)eps, dx, n, Cu, iu);
        else bn_bwd_dx_fixed_kernel<T, false, false><<<grid, blk, 0, c->stream>>>(dy, yact, var, gamma, (T)eps, dx, n, Cu, iu);
    }
    FX_LAUNCH_CHECK();
    return FX_OK;
}

}  // namespace

#define FX_DEFINE_BN(T, S)                                                                                             \
    extern "C" int fx_batchnorm_stats_##S(fx_ctx* c, const T* x, T* mean, T* var, T* running_mean, T* running_var,     \
                                          double momentum, int64_t outer, int64_t C, int64_t inner) {                  \
        return bn_stats<T>(c, x, mean, var, running_mean, running_var, momentum, outer, C, inner);                     \
    }                                                                                                                  \
    extern "C" int fx_batchnorm_fwd_##S(fx_ctx* c, const T* x, const T* mean, const T* var, const T* gamma,            \
                                        const T* beta, double eps, T* y, int64_t outer, int64_t C, int64_t inner,      \
                                        int act) {                                                                     \
        return bn_fwd<T>(c, x, mean, var, gamma, beta, eps, y, outer, C, inner, act);                                  \
    }                                                                                                                  \
    extern "C" int fx_batchnorm_bwd_##S(fx_ctx* c, const T* dy, const T* x, const T* y_act, const T* mean,             \
                                        const T* var, const T* gamma, double eps, T* dx, T* dgamma, T* dbeta,          \
                                        int64_t outer, int64_t C, int64_t inner, int batch_stats) {                    \
        return bn_bwd<T>(c, dy, x, y_act, mean, var, gamma, eps, dx, dgamma, dbeta, outer, C, inner, batch_stats);     \
    }

FX_DEFINE_BN(float, f32)
FX_DEFINE_BN(double, f64)
