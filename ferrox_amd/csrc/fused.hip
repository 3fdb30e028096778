// Fused entry points for sequences that the reference composes from many small operators; each keeps the
// composed path's arithmetic (same operations in the same order per element; this file is built without a*b+c
// contraction) so that results equal the composed path bit for bit wherever no reduction order is involved.
//   bias_act      y += bias[c] (then ReLU)      replaces Reshape + BroadcastTo + Add (+ ReLU): nn/layers/utils.rs:6-42,
//                                               conv2d.rs:203-213, linear.rs:262-279, ops/unary.rs:340-356
//   bias_grad     db[c] = sum_{o,i} g[o,c,i]    replaces reduce_gradient_for_broadcasting (ops/basic.rs:10-53)
//   softmax_ce    loss and d loss / d logits    replaces the 7 forward / 7 backward ops of CCELoss
//                                               (nn/losses/classification.rs:191-257, ops/batched.rs:106-131)
//   adam_step     in-place Adam update          replaces ~14 kernels per parameter (nn/optim/adam.rs:288-358)
//   sgd_step      in-place SGD update (plain, or with L2 weight decay / momentum / Nesterov)   replaces nn/optim/sgd.rs:128-245
//   adam_amsgrad  Adam with the running maximum of the second moment (adam.rs:203-221)
#include "common.hpp"

namespace {

template <typename T> __device__ __forceinline__ T dev_exp(T x);
template <> __device__ __forceinline__ float dev_exp<float>(float x) { return expf(x); }
template <> __device__ __forceinline__ double dev_exp<double>(double x) { return exp(x); }
template <typename T> __device__ __forceinline__ T dev_log(T x);
template <> __device__ __forceinline__ float dev_log<float>(float x) { return logf(x); }
template <> __device__ __forceinline__ double dev_log<double>(double x) { return log(x); }
template <typename T> __device__ __forceinline__ T dev_sqrt(T x);
template <> __device__ __forceinline__ float dev_sqrt<float>(float x) { return sqrtf(x); }
template <> __device__ __forceinline__ double dev_sqrt<double>(double x) { return sqrt(x); }
template <typename T> __device__ __forceinline__ T lowest();
template <> __device__ __forceinline__ float lowest<float>() { return -3.402823466e+38f; }
template <> __device__ __forceinline__ double lowest<double>() { return -1.7976931348623157e+308; }

// ---- bias add (+ ReLU), in place: y viewed as [outer, C, inner] ---------------------------------------------------
// VEC: inner is a multiple of the 16-byte vector and y is 16-byte aligned, so one thread owns one vector (one channel).
template <typename T, bool VEC, bool RELU>
__global__ __launch_bounds__(256) void bias_act_kernel(T* __restrict__ y, const T* __restrict__ bias, i64 n, uint32_t C, uint32_t inner) {
    constexpr int V = VEC ? 16 / (int)sizeof(T) : 1;
    typedef T vec_t __attribute__((ext_vector_type(V)));
    const i64 i = ((i64)blockIdx.x * 256 + threadIdx.x) * V;
    if (i >= n) return;
    const T b = bias[(i / inner) % C];
    vec_t v = *reinterpret_cast<vec_t*>(y + i);
#pragma unroll
    for (int u = 0; u < V; ++u) {
        T r = v[u] + b;
        if (RELU) r = r > T(0) ? r : T(0);  // ReLU as in the forward kernel: x > 0 ? x : 0
        v[u] = r;
    }
    *reinterpret_cast<vec_t*>(y + i) = v;
}

template <typename T>
int bias_act(fx_ctx* c, T* y, const T* bias, i64 outer, i64 C, i64 inner, int act) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(outer >= 0 && C >= 1 && inner >= 1, "fx_bias_act: bad view");
    FX_REQUIRE(act == 0 || act == 1, "fx_bias_act: act must be 0 (none) or 1 (relu)");
    const i64 n = outer * C * inner;
    if (n == 0) return FX_OK;
    FX_REQUIRE(y && bias, "fx_bias_act: null pointer");
    FX_REQUIRE(C < (1ll << 31) && inner < (1ll << 31), "fx_bias_act: view too large");
    constexpr int V = 16 / (int)sizeof(T);
    const bool vec = inner % V == 0 && ((uintptr_t)y & 15) == 0;
    const i64 threads = vec ? n / V : n, blocks = fx::ceil_div(threads, 256);
    FX_REQUIRE(blocks <= 0x7fffffff, "fx_bias_act: too many elements");
    const dim3 grid((unsigned)blocks), blk(256);
    if (vec) {
        if (act) bias_act_kernel<T, true, true><<<grid, blk, 0, c->stream>>>(y, bias, n, (uint32_t)C, (uint32_t)inner);
        else bias_act_kernel<T, true, false><<<grid, blk, 0, c->stream>>>(y, bias, n, (uint32_t)C, (uint32_t)inner);
    } else {
        if (act) bias_act_kernel<T, false, true><<<grid, blk, 0, c->stream>>>(y, bias, n, (uint32_t)C, (uint32_t)inner);
        else bias_act_kernel<T, false, false><<<grid, blk, 0, c->stream>>>(y, bias, n, (uint32_t)C, (uint32_t)inner);
    }
    FX_LAUNCH_CHECK();
    return FX_OK;
}

// ---- bias gradient: out[c] = sum over (o, i) of g[o, c, i] --------------------------------------------------------
// Stage 1: block (c, slice) sums rows o of its slice, each thread running over i and o in a fixed pattern, then a
// fixed-order tree; stage 2 adds the slice partials in slice order.  Deterministic for a given (outer, C, inner).
template <typename T>
__global__ __launch_bounds__(256) void bias_grad_partial_kernel(const T* __restrict__ g, T* __restrict__ part, i64 outer, i64 C,
                                                                i64 inner, i64 rows_per_slice) {
    __shared__ T sm[256];
    const i64 c = blockIdx.x, slice = blockIdx.y;
    const i64 o0 = slice * rows_per_slice, o1 = min(outer, o0 + rows_per_slice);
    T s = T(0);
    constexpr int V = 16 / (int)sizeof(T);
    typedef T vec_t __attribute__((ext_vector_type(V)));
    if (inner >= 64 && inner % V == 0 && ((uintptr_t)g & 15) == 0) {
        // threads run along i in 16-byte vectors, four rows in flight; one running sum per vector lane
        vec_t acc = vec_t(T(0));
        const i64 nv = inner / V;
        i64 o = o0;
        for (; o + 4 <= o1; o += 4) {
            for (i64 i = threadIdx.x; i < nv; i += 256) {
                vec_t v[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) v[u] = reinterpret_cast<const vec_t*>(g + ((o + u) * C + c) * inner)[i];
#pragma unroll
                for (int u = 0; u < 4; ++u) acc = acc + v[u];
            }
        }
        for (; o < o1; ++o)
            for (i64 i = threadIdx.x; i < nv; i += 256) acc = acc + reinterpret_cast<const vec_t*>(g + (o * C + c) * inner)[i];
#pragma unroll
        for (int u = 0; u < V; ++u) s = s + acc[u];
    } else if (inner >= 64) {  // threads run along i (contiguous), rows one after the other
        for (i64 o = o0; o < o1; ++o) {
            const T* p = g + (o * C + c) * inner;
            for (i64 i = threadIdx.x; i < inner; i += 256) s = s + p[i];
        }
    } else {  // short rows: threads run over (o, i) pairs
        const i64 total = (o1 - o0) * inner;
        for (i64 t = threadIdx.x; t < total; t += 256) {
            const i64 o = o0 + t / inner, i = t % inner;
            s = s + g[(o * C + c) * inner + i];
        }
    }
    sm[threadIdx.x] = s;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) {
        if ((int)threadIdx.x < w) sm[threadIdx.x] = sm[threadIdx.x] + sm[threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x == 0) part[slice * C + c] = sm[0];
}

// The same reduction fused with the ReLU gradient that precedes it in a conv / linear layer with a folded activation:
// gm = (y > 0 ? g : 0) is written out (the weight and data gradients read it) and summed per channel in one pass.
template <typename T>
__global__ __launch_bounds__(256) void relu_bias_grad_partial_kernel(const T* __restrict__ g, const T* __restrict__ y, T* __restrict__ gm,
                                                                     T* __restrict__ part, i64 outer, i64 C, i64 inner, i64 rows_per_slice) {
    __shared__ T sm[256];
    const i64 c = blockIdx.x, slice = blockIdx.y;
    const i64 o0 = slice * rows_per_slice, o1 = min(outer, o0 + rows_per_slice);
    T s = T(0);
    constexpr int V = 16 / (int)sizeof(T);
    typedef T vec_t __attribute__((ext_vector_type(V)));
    if (inner % V == 0 && ((uintptr_t)g & 15) == 0 && ((uintptr_t)y & 15) == 0 && ((uintptr_t)gm & 15) == 0) {
        // threads walk the (row, vector) pairs of the slice, so every thread is busy whatever `inner` is
        vec_t acc = vec_t(T(0));
        const i64 nv = inner / V, pairs = (o1 - o0) * nv;
        i64 o = o0 + threadIdx.x / nv, iv = threadIdx.x % nv;  // pair q = (row, vector); stepped without a division per load
        const i64 dq = 256 / nv, dr = 256 % nv;
        for (i64 q = threadIdx.x; q < pairs; q += 256) {
            const i64 off = (o * C + c) * inner + iv * V;
            o += dq;
            iv += dr;
            if (iv >= nv) { iv -= nv; ++o; }
            vec_t gv = *reinterpret_cast<const vec_t*>(g + off);
            const vec_t yv = *reinterpret_cast<const vec_t*>(y + off);
#pragma unroll
            for (int u = 0; u < V; ++u) gv[u] = gv[u] * (yv[u] > T(0) ? T(1) : T(0));  // ReluBwdF of the elementwise kernel
            *reinterpret_cast<vec_t*>(gm + off) = gv;
            acc = acc + gv;
        }
#pragma unroll
        for (int u = 0; u < V; ++u) s = s + acc[u];
    } else {
        const i64 total = (o1 - o0) * inner;
        for (i64 t = threadIdx.x; t < total; t += 256) {
            const i64 off = ((o0 + t / inner) * C + c) * inner + t % inner;
            const T v = g[off] * (y[off] > T(0) ? T(1) : T(0));
            gm[off] = v;
            s = s + v;
        }
    }
    sm[threadIdx.x] = s;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) {
        if ((int)threadIdx.x < w) sm[threadIdx.x] = sm[threadIdx.x] + sm[threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x == 0) part[slice * C + c] = sm[0];
}

template <typename T>
__global__ __launch_bounds__(256) void bias_grad_final_kernel(const T* __restrict__ part, T* __restrict__ out, i64 C, int slices) {
    const i64 c = (i64)blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    T s = T(0);
    for (int z = 0; z < slices; ++z) s = s + part[(i64)z * C + c];
    out[c] = s;
}

// y != nullptr: the fused ReLU-gradient form (gm receives the masked gradient)
template <typename T>
int bias_grad(fx_ctx* c, const T* g, T* out, i64 outer, i64 C, i64 inner, const T* y = nullptr, T* gm = nullptr) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(outer >= 1 && C >= 1 && inner >= 1, "fx_bias_grad: bad view");
    FX_REQUIRE(g && out && (y == nullptr) == (gm == nullptr), "fx_bias_grad: null pointer");
    FX_REQUIRE(C <= 0x7fffffff, "fx_bias_grad: too many channels");
    // enough blocks to fill the chip, at least 8 rows (or 16k elements) per block
    i64 slices = std::max<i64>(1, std::min<i64>((i64)c->num_cus * 4 / C, 65535));
    const i64 min_rows = std::max<i64>(1, 16384 / inner);
    slices = std::max<i64>(1, std::min<i64>(slices, outer / min_rows));
    const i64 rps = fx::ceil_div(outer, slices);
    slices = fx::ceil_div(outer, rps);
    std::lock_guard<std::mutex> lk(c->launch_mutex);
    T* part = out;
    if (slices > 1) {
        part = (T*)c->get_scratch(slices * C * (i64)sizeof(T));
        if (!part) return FX_ERR_OOM;
    }
    if (y) relu_bias_grad_partial_kernel<T><<<dim3((unsigned)C, (unsigned)slices), dim3(256), 0, c->stream>>>(g, y, gm, part, outer, C, inner, rps);
    else bias_grad_partial_kernel<T><<<dim3((unsigned)C, (unsigned)slices), dim3(256), 0, c->stream>>>(g, part, outer, C, inner, rps);
    FX_LAUNCH_CHECK();
    if (slices > 1) {
        bias_grad_final_kernel<T><<<dim3((unsigned)fx::ceil_div(C, (i64)256)), dim3(256), 0, c->stream>>>(part, out, C, (int)slices);
        FX_LAUNCH_CHECK();
    }
    return FX_OK;
}

// ---- softmax cross-entropy with mean reduction -------------------------------------------------------------------
// forward, one thread per row, classes walked in order (as softmax_batched and the row sum do):
//   s = exp(x - max) / sum;  p = clamp(s, 1e-8, 1 - 1e-8);  row = -(sum_c y*log(p));  loss = (sum_b row) * (1/B)
template <typename T>
__global__ __launch_bounds__(256) void softmax_ce_rows_kernel(const T* __restrict__ x, const T* __restrict__ y, T* __restrict__ probs,
                                                              T* __restrict__ rowloss, i64 B, i64 C, T lo, T hi) {
    const i64 b = (i64)blockIdx.x * 256 + threadIdx.x;
    if (b >= B) return;
    const T* xr = x + b * C;
    const T* yr = y + b * C;
    T* pr = probs + b * C;
    T m = lowest<T>();
    for (i64 k = 0; k < C; ++k) { const T v = xr[k]; if (v > m) m = v; }
    T s = T(0);
    for (i64 k = 0; k < C; ++k) { const T e = dev_exp<T>(xr[k] - m); pr[k] = e; s = s + e; }
    T acc = T(0);
    for (i64 k = 0; k < C; ++k) {
        const T sm = pr[k] / s;
        pr[k] = sm;
        T p = sm;
        if (p < lo) p = lo;
        if (p > hi) p = hi;
        acc = acc + yr[k] * dev_log<T>(p);
    }
    rowloss[b] = -acc;
}

template <typename T>
__global__ __launch_bounds__(256) void mean_rows_kernel(const T* __restrict__ rowloss, T* __restrict__ loss, i64 B, T inv) {
    __shared__ T sm[256];
    T s = T(0);
    for (i64 i = threadIdx.x; i < B; i += 256) s = s + rowloss[i];
    sm[threadIdx.x] = s;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) {
        if ((int)threadIdx.x < w) sm[threadIdx.x] = sm[threadIdx.x] + sm[threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x == 0) loss[0] = sm[0] * inv;
}

// Both steps in one block for small problems (up to 1024 rows and 16384 logits): thread t takes rows t, t + 256, ... -- the rows and the order in which
// mean_rows_kernel's thread t adds them -- and the same tree follows, so the loss has the bits of the two-kernel path.
// With dx != null the block also writes d loss / d logits for an upstream gradient of exactly 1 -- the operations of
// softmax_ce_bwd_kernel on the row it has just finished, in their order, so dx has that kernel's bits.
template <typename T>
__global__ __launch_bounds__(256) void softmax_ce_small_kernel(const T* __restrict__ x, const T* __restrict__ y, T* __restrict__ probs,
                                                               T* __restrict__ loss, T* __restrict__ dx, i64 B, i64 C, T lo, T hi, T inv) {
    __shared__ T sm[256];
    T tot = T(0);
    const T dtl = -(T(1) * inv);
    if (C <= 16) {
        // a row fits the registers: all of its loads are in flight together instead of one dependent access after the other
        // (the arithmetic and its order are those of the general loop below)
        const int c = (int)C;
        for (i64 b = threadIdx.x; b < B; b += 256) {
            T xv[16], yv[16], pv[16];
#pragma unroll
            for (int k = 0; k < 16; ++k) {
                xv[k] = k < c ? x[b * C + k] : T(0);
                yv[k] = k < c ? y[b * C + k] : T(0);
            }
            T m = lowest<T>();
#pragma unroll
            for (int k = 0; k < 16; ++k) if (k < c && xv[k] > m) m = xv[k];
            T s = T(0);
#pragma unroll
            for (int k = 0; k < 16; ++k) if (k < c) { pv[k] = dev_exp<T>(xv[k] - m); s = s + pv[k]; }
            T acc = T(0);
#pragma unroll
            for (int k = 0; k < 16; ++k) if (k < c) {
                const T smx = pv[k] / s;
                pv[k] = smx;
                T p = smx;
                if (p < lo) p = lo;
                if (p > hi) p = hi;
                acc = acc + yv[k] * dev_log<T>(p);
            }
#pragma unroll
            for (int k = 0; k < 16; ++k) if (k < c) probs[b * C + k] = pv[k];
            tot = tot + (-acc);
            if (dx) {
                T dv[16], dot = T(0);
#pragma unroll
                for (int k = 0; k < 16; ++k) if (k < c) {
                    const T sv = pv[k];
                    T p = sv;
                    if (p < lo) p = lo;
                    if (p > hi) p = hi;
                    const T dp = (dtl * yv[k]) / p;
                    const T ds = (dp * (sv >= lo ? T(1) : T(0))) * (sv <= hi ? T(1) : T(0));
                    dv[k] = ds;
                    dot = dot + ds * sv;
                }
#pragma unroll
                for (int k = 0; k < 16; ++k) if (k < c) dx[b * C + k] = pv[k] * (dv[k] - dot);
            }
        }
    } else
    for (i64 b = threadIdx.x; b < B; b += 256) {
        const T* xr = x + b * C;
        const T* yr = y + b * C;
        T* pr = probs + b * C;
        T m = lowest<T>();
        for (i64 k = 0; k < C; ++k) { const T v = xr[k]; if (v > m) m = v; }
        T s = T(0);
        for (i64 k = 0; k < C; ++k) { const T e = dev_exp<T>(xr[k] - m); pr[k] = e; s = s + e; }
        T acc = T(0);
        for (i64 k = 0; k < C; ++k) {
            const T smx = pr[k] / s;
            pr[k] = smx;
            T p = smx;
            if (p < lo) p = lo;
            if (p > hi) p = hi;
            acc = acc + yr[k] * dev_log<T>(p);
        }
        tot = tot + (-acc);
        if (dx) {
            T* dr = dx + b * C;
            T dot = T(0);
            for (i64 k = 0; k < C; ++k) {
                const T sv = pr[k];
                T p = sv;
                if (p < lo) p = lo;
                if (p > hi) p = hi;
                const T dp = (dtl * yr[k]) / p;
                const T ds = (dp * (sv >= lo ? T(1) : T(0))) * (sv <= hi ? T(1) : T(0));
                dr[k] = ds;
                dot = dot + ds * sv;
            }
            for (i64 k = 0; k < C; ++k) dr[k] = pr[k] * (dr[k] - dot);
        }
    }
    sm[threadIdx.x] = tot;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) {
        if ((int)threadIdx.x < w) sm[threadIdx.x] = sm[threadIdx.x] + sm[threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x == 0) loss[0] = sm[0] * inv;
}

template <typename T>
__global__ __launch_bounds__(256) void softmax_ce_bwd_kernel(const T* __restrict__ probs, const T* __restrict__ y, const T* __restrict__ gup,
                                                             T gval, T* __restrict__ dx, i64 B, i64 C, T inv, T lo, T hi);

// dlogits (optional): d loss / d logits for an upstream gradient of 1, with the bits of softmax_ce_bwd on a device 1.
template <typename T>
int softmax_ce_fwd(fx_ctx* c, const T* logits, const T* targets, T* probs, T* loss, i64 B, i64 C, T* dlogits = nullptr) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(B >= 1 && C >= 1, "fx_softmax_ce_fwd: bad shape");
    FX_REQUIRE(logits && targets && probs && loss, "fx_softmax_ce_fwd: null pointer");
    std::lock_guard<std::mutex> lk(c->launch_mutex);
    if (B <= 1024 && B * C <= 16384) {  // little work: one launch instead of two (or three)
        softmax_ce_small_kernel<T><<<dim3(1), dim3(256), 0, c->stream>>>(logits, targets, probs, loss, dlogits, B, C, (T)1e-8,
                                                                         (T)(1.0 - 1e-8), (T)(1.0 / (double)B));
        FX_LAUNCH_CHECK();
        return FX_OK;
    }

    T* rowloss = (T*)c->get_scratch(B * (i64)sizeof(T));
    if (!rowloss) return FX_ERR_OOM;
    softmax_ce_rows_kernel<T><<<dim3((unsigned)fx::ceil_div(B, (i64)256)), dim3(256), 0, c->stream>>>(
        logits, targets, probs, rowloss, B, C, (T)1e-8, (T)(1.0 - 1e-8));
    FX_LAUNCH_CHECK();
    mean_rows_kernel<T><<<dim3(1), dim3(256), 0, c->stream>>>(rowloss, loss, B, (T)(1.0 / (double)B));
    FX_LAUNCH_CHECK();
    if (dlogits) {
        softmax_ce_bwd_kernel<T><<<dim3((unsigned)fx::ceil_div(B, (i64)256)), dim3(256), 0, c->stream>>>(
            probs, targets, nullptr, T(1), dlogits, B, C, (T)(1.0 / (double)B), (T)1e-8, (T)(1.0 - 1e-8));
        FX_LAUNCH_CHECK();
    }
    return FX_OK;
}

// backward: upstream g (one element on the device) -> d logits, the composed chain evaluated per row:
//   d_tl = (-(g * (1/B)));  d_logp = d_tl * y;  d_p = d_logp / p;  d_s = d_p * (s >= lo) * (s <= hi);
//   d_x = s * (d_s - sum_c(d_s * s))
// The upstream gradient is gup[0], or gval where gup is null.
template <typename T>
__global__ __launch_bounds__(256) void softmax_ce_bwd_kernel(const T* __restrict__ probs, const T* __restrict__ y, const T* __restrict__ gup,
                                                             T gval, T* __restrict__ dx, i64 B, i64 C, T inv, T lo, T hi) {
    const i64 b = (i64)blockIdx.x * 256 + threadIdx.x;
    if (b >= B) return;
    const T* sr = probs + b * C;
    const T* yr = y + b * C;
    T* dr = dx + b * C;
    const T dtl = -((gup ? gup[0] : gval) * inv);
    T dot = T(0);
    if (C <= 16) {  // the row in registers, loads in flight together; same arithmetic in the same order as below
        const int c = (int)C;
        T sv[16], yv[16], dv[16];
#pragma unroll
        for (int k = 0; k < 16; ++k) {
            sv[k] = k < c ? sr[k] : T(0);
            yv[k] = k < c ? yr[k] : T(0);
        }
#pragma unroll
        for (int k = 0; k < 16; ++k) if (k < c) {
            const T s = sv[k];
            T p = s;
            if (p < lo) p = lo;
            if (p > hi) p = hi;
            const T dp = (dtl * yv[k]) / p;
            const T ds = (dp * (s >= lo ? T(1) : T(0))) * (s <= hi ? T(1) : T(0));
            dv[k] = ds;
            dot = dot + ds * s;
        }
#pragma unroll
        for (int k = 0; k < 16; ++k) if (k < c) dr[k] = sv[k] * (dv[k] - dot);
        return;
    }
    for (i64 k = 0; k < C; ++k) {
        const T s = sr[k];
        T p = s;
        if (p < lo) p = lo;
        if (p > hi) p = hi;
        const T dp = (dtl * yr[k]) / p;
        const T ds = (dp * (s >= lo ? T(1) : T(0))) * (s <= hi ? T(1) : T(0));
        dr[k] = ds;
        dot = dot + ds * s;
    }
    for (i64 k = 0; k < C; ++k) dr[k] = sr[k] * (dr[k] - dot);
}

template <typename T>
int softmax_ce_bwd(fx_ctx* c, const T* probs, const T* targets, const T* gup, T* dlogits, i64 B, i64 C) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(B >= 1 && C >= 1, "fx_softmax_ce_bwd: bad shape");
    FX_REQUIRE(probs && targets && gup && dlogits, "fx_softmax_ce_bwd: null pointer");
    softmax_ce_bwd_kernel<T><<<dim3((unsigned)fx::ceil_div(B, (i64)256)), dim3(256), 0, c->stream>>>(
        probs, targets, gup, T(0), dlogits, B, C, (T)(1.0 / (double)B), (T)1e-8, (T)(1.0 - 1e-8));
    FX_LAUNCH_CHECK();
    return FX_OK;
}

// ---- optimizers, in place ----------------------------------------------------------------------------------------
// Element updates in the composed kernels' operation order (this file is built without a*b+c contraction), so the
// results have the bits of the op-by-op path.
//   Adam  (nn/optim/adam.rs:136-358): m = m*b1 + g*(1-b1); v = v*b2 + (g*g)*(1-b2); AMSGrad: vmax = max(vmax, v)
//         (cpu.rs:717-739: a >= b ? a : b) and vmax takes v's place below; p = p - ((m/bc1)/(sqrt(v/bc2)+eps))*lr
//         [- p*(wd*lr)]
//   SGD   (nn/optim/sgd.rs:128-245): e = g [+ p*wd]; momentum != 0: buf = buf*mu + e, u = nesterov ? buf*mu + e : buf;
//         else u = e; p = p - u*lr
template <typename T> struct OptHyper {
    T lr, beta1, beta2, eps, wd, bc1, bc2;  // SGD: beta1 = momentum
    int flag;                               // Adam: amsgrad; SGD: nesterov
    const T* bc_dev = nullptr;              // Adam: when set, {bc1, bc2} are read from device memory instead
};

template <typename T>
__device__ __forceinline__ void adam_element(T* p, const T* g, T* m, T* v, T* vmax, i64 i, const OptHyper<T>& h) {
    const T gi = g[i], w = p[i];
    const T m1 = m[i] * h.beta1 + gi * (T(1) - h.beta1);
    T m2 = v[i] * h.beta2 + (gi * gi) * (T(1) - h.beta2);
    m[i] = m1;
    v[i] = m2;
    if (vmax) {
        const T old = vmax[i];
        m2 = old >= m2 ? old : m2;
        vmax[i] = m2;
    }
    const T denom = dev_sqrt<T>(m2 / h.bc2) + h.eps;
    const T update = ((m1 / h.bc1) / denom) * h.lr;
    T nw = w - update;
    if (h.wd != T(0)) nw = nw - w * (h.wd * h.lr);
    p[i] = nw;
}

template <typename T>
__device__ __forceinline__ void sgd_element(T* p, const T* g, T* buf, i64 i, const OptHyper<T>& h) {
    const T w = p[i];
    T e = g[i];
    if (h.wd != T(0)) e = e + w * h.wd;
    T u = e;
    if (buf) {  // momentum != 0
        const T b = buf[i] * h.beta1 + e;
        buf[i] = b;
        u = h.flag ? b * h.beta1 + e : b;
    }
    p[i] = w - u * h.lr;
}

// Every parameter of a model in one launch: the tensor table travels in the kernel arguments (no device-side
// table to upload); block b belongs to the tensor t with first[t] <= b < first[t+1].
constexpr int MULTI_MAX = 24;
template <typename T> struct MultiTensors {
    T* p[MULTI_MAX];
    const T* g[MULTI_MAX];
    T* m[MULTI_MAX];   // Adam: first moment; SGD: momentum buffer (null without momentum)
    T* v[MULTI_MAX];   // Adam: second moment
    T* x[MULTI_MAX];   // Adam with AMSGrad: running maximum of the second moment (null otherwise)
    i64 n[MULTI_MAX];
    unsigned first[MULTI_MAX + 1];
    int count;
};

template <typename T, bool ADAM>
__global__ __launch_bounds__(256) void multi_step_kernel(const MultiTensors<T> tt, const OptHyper<T> h) {
    int t = 0;
    while (t + 1 < tt.count && blockIdx.x >= tt.first[t + 1]) ++t;  // wave-uniform
    const i64 i = (i64)(blockIdx.x - tt.first[t]) * 256 + threadIdx.x;
    if (i >= tt.n[t]) return;
    if (ADAM) {
        if (h.bc_dev) {  // the step-dependent scalars of a recorded step: a graph repeats the kernel with the arguments of the recording
            OptHyper<T> hs = h;
            hs.bc1 = h.bc_dev[0];
            hs.bc2 = h.bc_dev[1];
            adam_element<T>(tt.p[t], tt.g[t], tt.m[t], tt.v[t], tt.x[t], i, hs);
        } else adam_element<T>(tt.p[t], tt.g[t], tt.m[t], tt.v[t], tt.x[t], i, h);
    } else sgd_element<T>(tt.p[t], tt.g[t], tt.m[t], i, h);
}

// m / v / x: tables that may be null as a whole (SGD without momentum; Adam without AMSGrad)
template <typename T, bool ADAM>
int multi_step(fx_ctx* c, int count, T* const* p, const T* const* g, T* const* m, T* const* v, T* const* x, const int64_t* n,
               const OptHyper<T>& h, const char* what) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(count >= 0, "%s: negative tensor count", what);
    FX_REQUIRE(count == 0 || (p && g && n && (!ADAM || (m && v))), "%s: null table", what);
    for (int base = 0; base < count; base += MULTI_MAX) {
        MultiTensors<T> tt;
        tt.count = 0;
        i64 blocks = 0;
        for (int k = base; k < count && k < base + MULTI_MAX; ++k) {
            FX_REQUIRE(n[k] >= 0, "%s: negative element count", what);
            if (n[k] == 0) continue;
            FX_REQUIRE(p[k] && g[k] && (!m || m[k]) && (!v || v[k]) && (!x || x[k]), "%s: null pointer in tensor %d", what, k);
            const int t = tt.count++;
            tt.p[t] = p[k]; tt.g[t] = g[k];
            tt.m[t] = m ? m[k] : nullptr; tt.v[t] = v ? v[k] : nullptr; tt.x[t] = x ? x[k] : nullptr;
            tt.n[t] = n[k];
            tt.first[t] = (unsigned)blocks;
            blocks += fx::ceil_div(n[k], (i64)256);
            FX_REQUIRE(blocks <= 0x7fffffff, "%s: too many elements", what);
        }
        if (tt.count == 0) continue;
        tt.first[tt.count] = (unsigned)blocks;
        multi_step_kernel<T, ADAM><<<dim3((unsigned)blocks), dim3(256), 0, c->stream>>>(tt, h);
        FX_LAUNCH_CHECK();
    }
    return FX_OK;
}

template <typename T>
int adam_hyper(OptHyper<T>& h, T lr, T beta1, T beta2, T eps, T wd, T bc1, T bc2, int amsgrad) {
    h.lr = lr; h.beta1 = beta1; h.beta2 = beta2; h.eps = eps; h.wd = wd; h.bc1 = bc1; h.bc2 = bc2; h.flag = amsgrad;
    return FX_OK;
}
template <typename T>
int sgd_hyper(OptHyper<T>& h, T lr, T momentum, T wd, int nesterov, bool have_buf, const char* what) {
    FX_REQUIRE((momentum != T(0)) == have_buf, "%s: a momentum buffer goes with a nonzero momentum, and only with one", what);
    h.lr = lr; h.beta1 = momentum; h.beta2 = T(0); h.eps = T(0); h.wd = wd; h.bc1 = T(1); h.bc2 = T(1); h.flag = nesterov;
    return FX_OK;
}

template <typename T>
int adam_step(fx_ctx* c, T* p, const T* g, T* m, T* v, T* vmax, i64 n, T lr, T beta1, T beta2, T eps, T wd, T bc1, T bc2, const char* what) {
    OptHyper<T> h;
    adam_hyper(h, lr, beta1, beta2, eps, wd, bc1, bc2, vmax != nullptr);
    return multi_step<T, true>(c, 1, &p, &g, &m, &v, vmax ? &vmax : nullptr, &n, h, what);
}

template <typename T>
int sgd_step(fx_ctx* c, T* p, const T* g, T* buf, i64 n, T lr, T momentum, T wd, int nesterov, const char* what) {
    OptHyper<T> h;
    if (int rc = sgd_hyper(h, lr, momentum, wd, nesterov, buf != nullptr, what)) return rc;
    return multi_step<T, false>(c, 1, &p, &g, buf ? &buf : nullptr, nullptr, nullptr, &n, h, what);
}

}  // namespace

#define FX_DEFINE_FUSED(T, S)                                                                                          \
    extern "C" int fx_bias_act_##S(fx_ctx* c, T* y, const T* bias, int64_t outer, int64_t C, int64_t inner, int act) { \
        return bias_act<T>(c, y, bias, outer, C, inner, act);                                                          \
    }                                                                                                                  \
    extern "C" int fx_bias_grad_##S(fx_ctx* c, const T* g, T* out, int64_t outer, int64_t C, int64_t inner) {          \
        return bias_grad<T>(c, g, out, outer, C, inner);                                                               \
    }                                                                                                                  \
    extern "C" int fx_relu_bwd_bias_grad_##S(fx_ctx* c, const T* g, const T* y, T* gm, T* dbias, int64_t outer,        \
                                             int64_t C, int64_t inner) {                                               \
        FX_REQUIRE(y && gm, "fx_relu_bwd_bias_grad: null pointer");                                                    \
        return bias_grad<T>(c, g, dbias, outer, C, inner, y, gm);                                                      \
    }                                                                                                                  \
    extern "C" int fx_softmax_ce_fwd_##S(fx_ctx* c, const T* logits, const T* targets, T* probs, T* loss, int64_t B,   \
                                         int64_t C) {                                                                  \
        return softmax_ce_fwd<T>(c, logits, targets, probs, loss, B, C);                                               \
    }                                                                                                                  \
    extern "C" int fx_softmax_ce_fwd_unit_grad_##S(fx_ctx* c, const T* logits, const T* targets, T* probs, T* loss,    \
                                                   T* dlogits, int64_t B, int64_t C) {                                  \
        FX_REQUIRE(dlogits, "fx_softmax_ce_fwd_unit_grad: null pointer");                                              \
        return softmax_ce_fwd<T>(c, logits, targets, probs, loss, B, C, dlogits);                                      \
    }                                                                                                                  \
    extern "C" int fx_softmax_ce_bwd_##S(fx_ctx* c, const T* probs, const T* targets, const T* gup, T* dlogits,        \
                                         int64_t B, int64_t C) {                                                       \
        return softmax_ce_bwd<T>(c, probs, targets, gup, dlogits, B, C);                                               \
    }                                                                                                                  \
    extern "C" int fx_adam_step_##S(fx_ctx* c, T* p, const T* g, T* m, T* v, int64_t n, T lr, T beta1, T beta2, T eps, \
                                    T wd, T bc1, T bc2) {                                                              \
        FX_REQUIRE(n == 0 || (p && g && m && v), "fx_adam_step: null pointer");                                        \
        return adam_step<T>(c, p, g, m, v, nullptr, n, lr, beta1, beta2, eps, wd, bc1, bc2, "fx_adam_step");           \
    }                                                                                                                  \
    extern "C" int fx_adam_amsgrad_step_##S(fx_ctx* c, T* p, const T* g, T* m, T* v, T* vmax, int64_t n, T lr, T beta1, \
                                            T beta2, T eps, T wd, T bc1, T bc2) {                                      \
        FX_REQUIRE(n == 0 || (p && g && m && v && vmax), "fx_adam_amsgrad_step: null pointer");                        \
        return adam_step<T>(c, p, g, m, v, vmax, n, lr, beta1, beta2, eps, wd, bc1, bc2, "fx_adam_amsgrad_step");      \
    }                                                                                                                  \
    extern "C" int fx_sgd_step_##S(fx_ctx* c, T* p, const T* g, int64_t n, T lr) {                                     \
        FX_REQUIRE(n == 0 || (p && g), "fx_sgd_step: null pointer");                                                   \
        return sgd_step<T>(c, p, g, nullptr, n, lr, T(0), T(0), 0, "fx_sgd_step");                                     \
    }                                                                                                                  \
    extern "C" int fx_sgd_momentum_step_##S(fx_ctx* c, T* p, const T* g, T* buf, int64_t n, T lr, T momentum,          \
                                            T weight_decay, int nesterov) {                                            \
        FX_REQUIRE(n == 0 || (p && g), "fx_sgd_momentum_step: null pointer");                                          \
        return sgd_step<T>(c, p, g, buf, n, lr, momentum, weight_decay, nesterov, "fx_sgd_momentum_step");             \
    }                                                                                                                  \
    extern "C" int fx_adam_step_multi_##S(fx_ctx* c, int count, T* const* p, const T* const* g, T* const* m,           \
                                          T* const* v, const int64_t* n, T lr, T beta1, T beta2, T eps, T wd, T bc1,   \
                                          T bc2) {                                                                     \
        OptHyper<T> h;                                                                                                 \
        adam_hyper(h, lr, beta1, beta2, eps, wd, bc1, bc2, 0);                                                         \
        return multi_step<T, true>(c, count, p, g, m, v, nullptr, n, h, "fx_adam_step_multi");                         \
    }                                                                                                                  \
    extern "C" int fx_adam_step_multi_bc_##S(fx_ctx* c, int count, T* const* p, const T* const* g, T* const* m,        \
                                              T* const* v, T* const* vmax, const int64_t* n, T lr, T beta1, T beta2,    \
                                              T eps, T wd, const T* bc) {                                              \
        FX_REQUIRE(bc != nullptr, "fx_adam_step_multi_bc: null bias-correction pointer");                             \
        OptHyper<T> h;                                                                                                 \
        adam_hyper(h, lr, beta1, beta2, eps, wd, T(1), T(1), vmax != nullptr);                                         \
        h.bc_dev = bc;                                                                                                 \
        return multi_step<T, true>(c, count, p, g, m, v, vmax, n, h, "fx_adam_step_multi_bc");                         \
    }                                                                                                                  \
    extern "C" int fx_adam_amsgrad_step_multi_##S(fx_ctx* c, int count, T* const* p, const T* const* g, T* const* m,   \
                                                  T* const* v, T* const* vmax, const int64_t* n, T lr, T beta1,        \
                                                  T beta2, T eps, T wd, T bc1, T bc2) {                                \
        FX_REQUIRE(count == 0 || vmax, "fx_adam_amsgrad_step_multi: null table");                                      \
        OptHyper<T> h;                                                                                                 \
        adam_hyper(h, lr, beta1, beta2, eps, wd, bc1, bc2, 1);                                                         \
        return multi_step<T, true>(c, count, p, g, m, v, vmax, n, h, "fx_adam_amsgrad_step_multi");                    \
    }                                                                                                                  \
    extern "C" int fx_sgd_step_multi_##S(fx_ctx* c, int count, T* const* p, const T* const* g, const int64_t* n,       \
                                         T lr) {                                                                       \
        OptHyper<T> h;                                                                                                 \
        sgd_hyper(h, lr, T(0), T(0), 0, false, "fx_sgd_step_multi");                                                   \
        return multi_step<T, false>(c, count, p, g, nullptr, nullptr, nullptr, n, h, "fx_sgd_step_multi");             \
    }                                                                                                                  \
    extern "C" int fx_sgd_momentum_step_multi_##S(fx_ctx* c, int count, T* const* p, const T* const* g, T* const* buf, \
                                                  const int64_t* n, T lr, T momentum, T weight_decay, int nesterov) {  \
        FX_REQUIRE(count == 0 || (momentum != T(0)) == (buf != nullptr),                                               \
                   "fx_sgd_momentum_step_multi: a momentum buffer table goes with a nonzero momentum, and only with one"); \
        OptHyper<T> h;                                                                                                 \
        sgd_hyper(h, lr, momentum, weight_decay, nesterov, momentum != T(0), "fx_sgd_momentum_step_multi");            \
        return multi_step<T, false>(c, count, p, g, buf, nullptr, nullptr, n, h, "fx_sgd_momentum_step_multi");        \
    }

FX_DEFINE_FUSED(float, f32)
FX_DEFINE_FUSED(double, f64)
