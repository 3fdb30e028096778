// TEST INFRASTRUCTURE ONLY. This file is the CPU oracle: a single-thread restatement of the
// Ferrox CPU (ndarray) backend for the training hot path. Only tests, the smoke check and
// the benchmark's cpu_baseline leg may load it; the product library never links or calls it.
//
// Every function cites the reference file:line (relative to the Ferrox repository root) that
// it follows. Compile with -ffp-contract=off: Rust never contracts a*b+c into an fma, and the
// bit-exact claims (im2col/col2im layout and accumulation order, max/argmax) rely on that.
//
// Parity status of each part (what pins it besides this restatement):
//   im2col, col2im(layout 0/1)    : closed form + brute force + window-count identities (tests/test_oracle_*.py)
//   conv2d forward                : reference-held PyTorch vector src/ops/mod.rs:743-801 and torch CPU conv2d
//   conv2d dgrad/wgrad "correct"  : torch.autograd of conv2d (equals the reference CUDA kernels)
//   conv2d dgrad/wgrad "literal"  : for batch > 1, rebuilt from independent routines: numpy float64 matmul on the flat
//                                   [Cout, B*L] re-read of grad_output, torch unfold as im2col, torch fold on the
//                                   batch-major [B, C*kh*kw, L] re-read of the column matrix (the two re-reads are
//                                   the only thing taken from convolutions.rs:122-127, 292-293, 323-326); equality
//                                   with the correct mode at batch 1 and, for the weight gradient, at Cout = 1
//   gemm                          : 2x2 vectors src/ops/mod.rs:516-529, numpy float64 matmul
//   reductions                    : 2x2 vectors src/ops/mod.rs:544-618, numpy; summation ORDER at real
//                                   sizes is PARITY UNPINNED (ndarray/matrixmultiply sources are not in the
//                                   reference tree), compared by tolerance against float64 ground truth
//   activations fwd/bwd           : src/ops/mod.rs:480-506 vectors, libm closed forms, finite differences
//   softmax                       : src/ops/mod.rs:695-721 vectors
//   allocator                     : scripted traces with hand-computed counters (tests/test_pool_oracle.py)
#include <cstdint>
#include <cstring>
#include <cmath>
#include <cfloat>
#include <vector>
#include <algorithm>
#include <limits>

typedef int64_t i64;

// Fast single-thread GEMM lives in oracle_gemm.cpp (compiled with contraction allowed; stands in for
// matrixmultiply 0.3.10, whose summation order cannot be reproduced here).
template <typename T>
void orc_gemm_fast(int ta, int tb, i64 M, i64 N, i64 K, const T* A, const T* B, T* C);

namespace {

// ---------------------------------------------------------------------------------------------
// im2col: src/backend/storage/extensions/convolutions.rs:10-75
// col[(c*kh*kw + ky*kw + kx) * (B*oh*ow) + (b*oh*ow + oy*ow + ox)] = x[b,c,oy*sh+ky-ph, ox*sw+kx-pw] or 0.
// ---------------------------------------------------------------------------------------------
template <typename T>
void im2col(const T* x, i64 B, i64 C, i64 H, i64 W, i64 kh, i64 kw, i64 sh, i64 sw, i64 ph, i64 pw, T* col) {
    const i64 oh = (H + 2 * ph - kh) / sh + 1;
    const i64 ow = (W + 2 * pw - kw) / sw + 1;
    const i64 col_w = B * oh * ow;
    std::fill(col, col + C * kh * kw * col_w, T(0));
    for (i64 b = 0; b < B; ++b)
        for (i64 c = 0; c < C; ++c)
            for (i64 ky = 0; ky < kh; ++ky)
                for (i64 kx = 0; kx < kw; ++kx) {
                    const i64 row = c * kh * kw + ky * kw + kx;
                    for (i64 oy = 0; oy < oh; ++oy)
                        for (i64 ox = 0; ox < ow; ++ox) {
                            const i64 iy = oy * sh + ky, ix = ox * sw + kx;
                            if (iy >= ph && iy < H + ph && ix >= pw && ix < W + pw) {
                                const i64 ay = iy - ph, ax = ix - pw;
                                col[row * col_w + b * oh * ow + oy * ow + ox] = x[((b * C + c) * H + ay) * W + ax];
                            }
                        }
                }
}

// ---------------------------------------------------------------------------------------------
// col2im: src/backend/storage/extensions/convolutions.rs:79-153
// layout 1 ("literal"): the reference reads the column matrix with a batch-major flat index
//   b*(C*kh*kw*L) + c*(kh*kw*L) + ky*(kw*L) + kx*L + cy*cw + cx            (:122-127)
// layout 0 ("rowmajor"): the index that matches what im2col/GEMM actually produce,
//   (c*kh*kw + ky*kw + kx) * (B*L) + b*L + cy*cw + cx.
// Both accumulate into a zeroed padded image in the loop order (b, c, ky, kx, cy, cx) and crop.
// ---------------------------------------------------------------------------------------------
template <typename T>
void col2im(const T* col, i64 B, i64 C, i64 H, i64 W, i64 kh, i64 kw, i64 sh, i64 sw, i64 ph, i64 pw, T* out,
            int layout) {
    const i64 PH = H + 2 * ph, PW = W + 2 * pw;
    const i64 ch = (PH - kh) / sh + 1, cw = (PW - kw) / sw + 1;
    const i64 L = ch * cw;
    std::vector<T> padded((size_t)(B * C * PH * PW), T(0));
    for (i64 b = 0; b < B; ++b)
        for (i64 c = 0; c < C; ++c)
            for (i64 ky = 0; ky < kh; ++ky)
                for (i64 kx = 0; kx < kw; ++kx)
                    for (i64 cy = 0; cy < ch; ++cy)
                        for (i64 cx = 0; cx < cw; ++cx) {
                            const i64 iy = cy * sh + ky, ix = cx * sw + kx;
                            i64 idx;
                            if (layout == 1)
                                idx = b * (C * kh * kw * L) + c * (kh * kw * L) + ky * (kw * L) + kx * L + cy * cw + cx;
                            else
                                idx = (c * kh * kw + ky * kw + kx) * (B * L) + b * L + cy * cw + cx;
                            padded[((b * C + c) * PH + iy) * PW + ix] += col[idx];
                        }
    for (i64 b = 0; b < B; ++b)
        for (i64 c = 0; c < C; ++c)
            for (i64 h = 0; h < H; ++h)
                for (i64 w = 0; w < W; ++w)
                    out[((b * C + c) * H + h) * W + w] = padded[((b * C + c) * PH + h + ph) * PW + w + pw];
}

// transpose_conv_output: convolutions.rs:156-185   [OC, B*L] -> [B, OC, L]
template <typename T>
void transpose_conv_output(const T* src, i64 B, i64 OC, i64 L, T* dst) {
    for (i64 oc = 0; oc < OC; ++oc)
        for (i64 b = 0; b < B; ++b)
            for (i64 l = 0; l < L; ++l) dst[(b * OC + oc) * L + l] = src[oc * (B * L) + b * L + l];
}

// Naive GEMM, sequential k accumulation in T. Used for tiny fixtures only.
template <typename T>
void gemm_naive(int ta, int tb, i64 M, i64 N, i64 K, const T* A, const T* Bm, T* Cm) {
    for (i64 m = 0; m < M; ++m)
        for (i64 n = 0; n < N; ++n) {
            T acc = T(0);
            for (i64 k = 0; k < K; ++k) {
                const T a = ta ? A[k * M + m] : A[m * K + k];
                const T b = tb ? Bm[n * K + k] : Bm[k * N + n];
                acc += a * b;
            }
            Cm[m * N + n] = acc;
        }
}

// conv2d_impl: convolutions.rs:218-265  (im2col, flat copies elided, W2d . col, transpose back)
template <typename T>
void conv2d_fwd(const T* x, const T* w, T* y, i64 B, i64 Cin, i64 H, i64 W, i64 Cout, i64 kh, i64 kw, i64 sh, i64 sw,
                i64 ph, i64 pw) {
    const i64 oh = (H + 2 * ph - kh) / sh + 1, ow = (W + 2 * pw - kw) / sw + 1;
    const i64 K = Cin * kh * kw, N = B * oh * ow;
    std::vector<T> col((size_t)(K * N)), y2((size_t)(Cout * N));
    im2col(x, B, Cin, H, W, kh, kw, sh, sw, ph, pw, col.data());
    orc_gemm_fast<T>(0, 0, Cout, N, K, w, col.data(), y2.data());
    transpose_conv_output(y2.data(), B, Cout, oh * ow, y);
}

// deconv2d_impl: convolutions.rs:268-307.  g is [B, OC, oh, ow]; result is [B, Cin, H, W].
// mode 1 (literal): G2d = flat reinterpretation of g as [OC, B*L] (:292-293), col = W2d^T . G2d, col2im layout 1.
// mode 0 (correct): G2d[oc, b*L+l] = g[b,oc,l] (a true [B,OC]->[OC,B] transpose), col2im layout 0. This is the
//                   mathematical data gradient, equal to the reference CUDA kernel kernels/convolutions.cu:360-438.
template <typename T>
void conv2d_dgrad(const T* g, const T* w, T* dx, i64 B, i64 Cin, i64 H, i64 W, i64 Cout, i64 kh, i64 kw, i64 sh,
                  i64 sw, i64 ph, i64 pw, int mode) {
    const i64 oh = (H + 2 * ph - kh) / sh + 1, ow = (W + 2 * pw - kw) / sw + 1;
    const i64 L = oh * ow, K = Cin * kh * kw, N = B * L;
    std::vector<T> g2;
    const T* G2 = g;
    if (mode == 0) {
        g2.resize((size_t)(Cout * N));
        for (i64 b = 0; b < B; ++b)
            for (i64 oc = 0; oc < Cout; ++oc)
                std::memcpy(&g2[(size_t)(oc * N + b * L)], &g[(b * Cout + oc) * L], sizeof(T) * L);
        G2 = g2.data();
    }
    std::vector<T> col((size_t)(K * N));
    // col[K, N] = W2d^T[K, OC] . G2d[OC, N]  ; W2d is [OC, K] row-major -> transA
    orc_gemm_fast<T>(1, 0, K, N, Cout, w, G2, col.data());
    col2im(col.data(), B, Cin, H, W, kh, kw, sh, sw, ph, pw, dx, mode == 1 ? 1 : 0);
}

// cross_correlation2d_impl: convolutions.rs:310-338.  dW2d[OC, K] = G2d[OC, N] . col^T, col = im2col(x).
// mode 1 (literal): G2d = flat reinterpretation of g (:323-326).  mode 0 (correct): true transpose.
template <typename T>
void conv2d_wgrad(const T* x, const T* g, T* dw, i64 B, i64 Cin, i64 H, i64 W, i64 Cout, i64 kh, i64 kw, i64 sh,
                  i64 sw, i64 ph, i64 pw, int mode) {
    const i64 oh = (H + 2 * ph - kh) / sh + 1, ow = (W + 2 * pw - kw) / sw + 1;
    const i64 L = oh * ow, K = Cin * kh * kw, N = B * L;
    std::vector<T> col((size_t)(K * N));
    im2col(x, B, Cin, H, W, kh, kw, sh, sw, ph, pw, col.data());
    std::vector<T> g2;
    const T* G2 = g;
    if (mode == 0) {
        g2.resize((size_t)(Cout * N));
        for (i64 b = 0; b < B; ++b)
            for (i64 oc = 0; oc < Cout; ++oc)
                std::memcpy(&g2[(size_t)(oc * N + b * L)], &g[(b * Cout + oc) * L], sizeof(T) * L);
        G2 = g2.data();
    }
    // dW[OC, K] = G2[OC, N] . col[K, N]^T  -> transB
    orc_gemm_fast<T>(0, 1, Cout, K, N, G2, col.data(), dw);
}

// ---------------------------------------------------------------------------------------------
// Elementwise: src/backend/storage/cpu.rs:629-690 (binary), :741-767 (scalar, neg), :792-813 (clamp, sqrt),
// :829-918 (comparisons -> 1.0/0.0), :1004-1016 sigmoid, :1070-1100 relu/exp/log, :1102-1150 tanh.
// ---------------------------------------------------------------------------------------------
enum { B_ADD = 0, B_SUB = 1, B_MUL = 2, B_DIV = 3, B_EQUAL = 4, B_GREATER = 5, B_GE = 6, B_LESS = 7, B_LE = 8, B_MIN = 9, B_MAX = 10, B_POW = 11 };
enum { U_NEG = 0, U_SQRT = 1, U_EXP = 2, U_LOG = 3, U_RELU = 4, U_SIGMOID = 5, U_TANH = 6, U_ABS = 7, U_RECIP = 8, U_SIGN = 9, U_NOT = 10 };
enum { S_ADD = 0, S_SUB = 1, S_MUL = 2, S_DIV = 3, S_GREATER = 4, S_GE = 5, S_LE = 6, S_LESS = 7, S_POW = 8 };

template <typename T>
T tanh_ref(T x) {  // cpu.rs:1108-1147
    if (x > T(20.0)) return T(1);
    if (x < T(-20.0)) return T(-1);
    if (x >= T(0)) {
        const T e = std::exp(-x * T(2.0));
        const T num = T(1) - e, den = T(1) + e;
        return den == T(0) ? T(1) : num / den;
    }
    const T e = std::exp(x * T(2.0));
    const T num = e - T(1), den = e + T(1);
    return den == T(0) ? T(-1) : num / den;
}

template <typename T>
void binary(int op, const T* a, const T* b, T* o, i64 n) {
    for (i64 i = 0; i < n; ++i) {
        const T x = a[i], y = b[i];
        T r;
        switch (op) {
            case B_ADD: r = x + y; break;
            case B_SUB: r = x - y; break;
            case B_MUL: r = x * y; break;
            case B_DIV: r = x / y; break;
            case B_EQUAL: r = x == y ? T(1) : T(0); break;
            case B_GREATER: r = x > y ? T(1) : T(0); break;
            case B_GE: r = x >= y ? T(1) : T(0); break;
            case B_LESS: r = x < y ? T(1) : T(0); break;
            case B_LE: r = x <= y ? T(1) : T(0); break;
            case B_MIN: r = x <= y ? x : y; break;   // cpu.rs:708
            case B_MAX: r = x >= y ? x : y; break;   // cpu.rs:732
            case B_POW: r = std::pow(x, y); break;   // cpu.rs:1152-1172
            default: r = T(0);
        }
        o[i] = r;
    }
}

template <typename T>
void scalar_op(int op, const T* a, T s, T* o, i64 n) {
    for (i64 i = 0; i < n; ++i) {
        const T x = a[i];
        T r;
        switch (op) {
            case S_ADD: r = x + s; break;
            case S_SUB: r = x - s; break;
            case S_MUL: r = x * s; break;
            case S_DIV: r = x / s; break;
            case S_GREATER: r = x > s ? T(1) : T(0); break;
            case S_GE: r = x >= s ? T(1) : T(0); break;
            case S_LE: r = x <= s ? T(1) : T(0); break;
            case S_LESS: r = x < s ? T(1) : T(0); break;
            case S_POW: r = std::pow(x, s); break;   // cpu.rs:1174-1181
            default: r = T(0);
        }
        o[i] = r;
    }
}

template <typename T>
void unary(int op, const T* a, T* o, i64 n) {
    for (i64 i = 0; i < n; ++i) {
        const T x = a[i];
        T r;
        switch (op) {
            case U_NEG: r = -x; break;
            case U_SQRT: r = std::sqrt(x); break;
            case U_EXP: r = std::exp(x); break;
            case U_LOG: r = std::log(x); break;
            case U_RELU: r = x > T(0) ? x : T(0); break;             // cpu.rs:1072-1079
            case U_SIGMOID: r = T(1) / (T(1) + std::exp(-x)); break;  // cpu.rs:1009-1013
            case U_TANH: r = tanh_ref(x); break;
            case U_ABS: r = std::fabs(x); break;
            case U_RECIP: r = T(1) / x; break;
            case U_SIGN: r = x > T(0) ? T(1) : (x < T(0) ? -T(1) : T(0)); break;  // cpu.rs:949-965
            case U_NOT: r = x == T(0) ? T(1) : T(0); break;                       // cpu.rs:920-931
            default: r = T(0);
        }
        o[i] = r;
    }
}

template <typename T>
void clamp(const T* a, T lo, T hi, T* o, i64 n) {  // cpu.rs:792-805
    for (i64 i = 0; i < n; ++i) {
        const T x = a[i];
        o[i] = x < lo ? lo : (x > hi ? hi : x);
    }
}

// Activation backward, as the operator layer composes it from storage ops (each step rounds to T):
//   ReLU   src/ops/unary.rs:358-375 : g * (x > 0 ? 1 : 0)
//   Sigmoid src/ops/unary.rs:254-276: local = s * (s - 1)   [literal: note the sign]; g * local
//                                     mode 0 ("correct"): local = s * (1 - s)
//   Tanh   src/ops/unary.rs:306-328 : local = -((t*t) - 1); g * local
template <typename T>
void relu_bwd(const T* g, const T* x, T* o, i64 n) {
    for (i64 i = 0; i < n; ++i) o[i] = g[i] * (x[i] > T(0) ? T(1) : T(0));
}
template <typename T>
void sigmoid_bwd(const T* g, const T* s, T* o, i64 n, int literal) {
    for (i64 i = 0; i < n; ++i) {
        const T t = literal ? (s[i] - T(1)) : (T(1) - s[i]);
        const T local = s[i] * t;
        o[i] = g[i] * local;
    }
}
template <typename T>
void tanh_bwd(const T* g, const T* t, T* o, i64 n) {
    for (i64 i = 0; i < n; ++i) {
        const T sq = t[i] * t[i];
        const T m = sq - T(1);
        o[i] = g[i] * (-m);
    }
}

// ---------------------------------------------------------------------------------------------
// Reductions along one axis of a contiguous [outer, axis, inner] view: cpu.rs:60-130, 1183-1238.
// Summation order follows what ndarray 0.16 is believed to do (source not in the reference tree):
//  inner == 1  -> each lane is summed with an 8-accumulator unrolled fold;
//  inner  > 1  -> running sum of the sub-views in axis order.
// Max: in-order fold from T::MIN with a strict '>' (cpu.rs:1231-1234); argmax = first index that
// attains it (index 0 if nothing exceeds T::MIN).
// ---------------------------------------------------------------------------------------------
template <typename T>
T lane_sum_unrolled(const T* xs, i64 n) {
    T acc = T(0), p0 = T(0), p1 = T(0), p2 = T(0), p3 = T(0), p4 = T(0), p5 = T(0), p6 = T(0), p7 = T(0);
    while (n >= 8) {
        p0 = p0 + xs[0]; p1 = p1 + xs[1]; p2 = p2 + xs[2]; p3 = p3 + xs[3];
        p4 = p4 + xs[4]; p5 = p5 + xs[5]; p6 = p6 + xs[6]; p7 = p7 + xs[7];
        xs += 8; n -= 8;
    }
    acc = acc + (p0 + p4);
    acc = acc + (p1 + p5);
    acc = acc + (p2 + p6);
    acc = acc + (p3 + p7);
    for (i64 i = 0; i < n; ++i) acc = acc + xs[i];
    return acc;
}

template <typename T>
void reduce_sum_axis(const T* x, i64 outer, i64 axis, i64 inner, T* out) {
    if (inner == 1) {
        for (i64 o = 0; o < outer; ++o) out[o] = lane_sum_unrolled(x + o * axis, axis);
        return;
    }
    for (i64 o = 0; o < outer; ++o) {
        T* r = out + o * inner;
        for (i64 i = 0; i < inner; ++i) r[i] = T(0);
        for (i64 a = 0; a < axis; ++a) {
            const T* s = x + (o * axis + a) * inner;
            for (i64 i = 0; i < inner; ++i) r[i] = r[i] + s[i];
        }
    }
}

template <typename T>
void reduce_max_axis(const T* x, i64 outer, i64 axis, i64 inner, T* out, i64* idx) {
    const T lowest = std::numeric_limits<T>::lowest();  // FerroxN::min_value, number.rs:234-236, 357-359
    for (i64 o = 0; o < outer; ++o)
        for (i64 i = 0; i < inner; ++i) {
            T acc = lowest;
            i64 am = 0;
            for (i64 a = 0; a < axis; ++a) {
                const T v = x[(o * axis + a) * inner + i];
                if (v > acc) { acc = v; am = a; }
            }
            out[o * inner + i] = acc;
            if (idx) idx[o * inner + i] = am;
        }
}

// softmax_batched: cpu.rs:1037-1068
template <typename T>
void softmax_axis(const T* x, i64 outer, i64 axis, i64 inner, T* out) {
    std::vector<T> mx((size_t)(outer * inner)), sm((size_t)(outer * inner));
    reduce_max_axis(x, outer, axis, inner, mx.data(), (i64*)nullptr);
    for (i64 o = 0; o < outer; ++o)
        for (i64 a = 0; a < axis; ++a)
            for (i64 i = 0; i < inner; ++i) {
                const i64 p = (o * axis + a) * inner + i;
                out[p] = std::exp(x[p] - mx[o * inner + i]);
            }
    reduce_sum_axis(out, outer, axis, inner, sm.data());
    for (i64 o = 0; o < outer; ++o)
        for (i64 a = 0; a < axis; ++a)
            for (i64 i = 0; i < inner; ++i) {
                const i64 p = (o * axis + a) * inner + i;
                out[p] = out[p] / sm[o * inner + i];
            }
}

template <typename T>
void reduce_min_axis(const T* x, i64 outer, i64 axis, i64 inner, T* out, i64* idx) {  // cpu.rs:1240-1252
    const T highest = std::numeric_limits<T>::max();  // FerroxN::max_value
    for (i64 o = 0; o < outer; ++o)
        for (i64 i = 0; i < inner; ++i) {
            T acc = highest;
            i64 am = 0;
            for (i64 a = 0; a < axis; ++a) {
                const T v = x[(o * axis + a) * inner + i];
                if (v < acc) { acc = v; am = a; }
            }
            out[o * inner + i] = acc;
            if (idx) idx[o * inner + i] = am;
        }
}

// Product along the axis, from 1, positions in increasing order.  The reference has no CPU product; this restates the
// per-output arithmetic of kernels/reduction.cu:263-301 (prod = 1; prod *= input[...]) without its 32-lane tree, so
// the device result is compared to tolerance, never bit for bit.
template <typename T>
void reduce_prod_axis(const T* x, i64 outer, i64 axis, i64 inner, T* out) {
    for (i64 o = 0; o < outer; ++o)
        for (i64 i = 0; i < inner; ++i) {
            T acc = T(1);
            for (i64 a = 0; a < axis; ++a) acc = acc * x[(o * axis + a) * inner + i];
            out[o * inner + i] = acc;
        }
}

template <typename T>
void in_range(const T* a, T lo, T hi, T* o, i64 n) {  // cpu.rs:933-947
    for (i64 i = 0; i < n; ++i) o[i] = (a[i] >= lo && a[i] <= hi) ? T(1) : T(0);
}

// pool2d_impl, extensions/pooling.rs:154-229 with MaxPoolOp / AvgPoolOp (:25-64); separate window / stride / padding
// per dimension so that the 1-D variant (:231-287) is H = 1 with a 1 x k window.
template <typename T>
void pool2d(const T* in, T* out, i64 N, i64 C, i64 H, i64 W, i64 kh, i64 kw, i64 sh, i64 sw, i64 ph, i64 pw, int is_max) {
    const i64 oh = (H + 2 * ph - kh) / sh + 1, ow = (W + 2 * pw - kw) / sw + 1;
    for (i64 b = 0; b < N; ++b)
        for (i64 c = 0; c < C; ++c)
            for (i64 oy = 0; oy < oh; ++oy)
                for (i64 ox = 0; ox < ow; ++ox) {
                    const i64 hs = oy * sh - ph, ws = ox * sw - pw;
                    T acc = is_max ? std::numeric_limits<T>::lowest() : T(0);
                    int count = 0;
                    for (i64 ky = 0; ky < kh; ++ky)
                        for (i64 kx = 0; kx < kw; ++kx) {
                            const i64 y = hs + ky, x = ws + kx;
                            if (y >= 0 && y < H && x >= 0 && x < W) {
                                const T v = in[((b * C + c) * H + y) * W + x];
                                if (is_max) { if (v > acc) acc = v; }
                                else { acc += v; count += 1; }
                            }
                        }
                    if (!is_max) acc = count > 0 ? acc / (T)count : T(0);
                    out[((b * C + c) * oh + oy) * ow + ox] = acc;
                }
}

// unpool2d_impl, extensions/pooling.rs:339-418 with MaxUnpoolOp / AvgUnpoolOp (:88-148): for every input position a
// scan over ALL output windows in (out_h, out_w) order, as the reference does.
template <typename T>
void unpool2d(const T* gout, const T* in, const T* pooled, T* gin, i64 N, i64 C, i64 H, i64 W, i64 kh, i64 kw, i64 sh, i64 sw,
              i64 ph, i64 pw, int is_max) {
    const i64 oh = (H + 2 * ph - kh) / sh + 1, ow = (W + 2 * pw - kw) / sw + 1;
    const float kernel_area = (float)(kh * kw);
    const T eps = (T)1e-8f;                      // FerroxN::from_f32(1e-8)
    const T scale = (T)(1.0f / kernel_area);     // FerroxN::from_f32(1.0 / kernel_area)
    for (i64 b = 0; b < N; ++b)
        for (i64 c = 0; c < C; ++c)
            for (i64 y = 0; y < H; ++y)
                for (i64 x = 0; x < W; ++x) {
                    const i64 ii = ((b * C + c) * H + y) * W + x;
                    T acc = T(0);
                    for (i64 oy = 0; oy < oh; ++oy)
                        for (i64 ox = 0; ox < ow; ++ox) {
                            const i64 hs = oy * sh - ph, ws = ox * sw - pw;
                            if (y >= hs && y < hs + kh && x >= ws && x < ws + kw) {
                                const i64 oi = ((b * C + c) * oh + oy) * ow + ox;
                                if (is_max) {
                                    const T o = in[ii], pv = pooled[oi];
                                    const T diff = o > pv ? o - pv : pv - o;
                                    if (diff < eps) acc += gout[oi];
                                } else {
                                    acc += gout[oi] * scale;
                                }
                            }
                        }
                    gin[ii] = acc;
                }
}

// materialize a strided/broadcast view into contiguous memory: cpu.rs:510-562 (broadcast_to, transpose -> to_owned)
template <typename T>
void materialize(const T* x, T* out, const i64* shape, const i64* strides, int ndim, i64 n) {
    for (i64 i = 0; i < n; ++i) {
        i64 r = i, off = 0;
        for (int d = ndim - 1; d >= 0; --d) {
            const i64 c = r % shape[d];
            r /= shape[d];
            off += c * strides[d];
        }
        out[i] = x[off];
    }
}

}  // namespace

// ---------------------------------------------------------------------------------------------
// C entry points (loaded with ctypes by the tests).
// ---------------------------------------------------------------------------------------------
#define ORC_INSTANTIATE(T, S)                                                                                         \
    extern "C" void orc_im2col_##S(const T* x, i64 B, i64 C, i64 H, i64 W, i64 kh, i64 kw, i64 sh, i64 sw, i64 ph,    \
                                   i64 pw, T* col) {                                                                   \
        im2col<T>(x, B, C, H, W, kh, kw, sh, sw, ph, pw, col);                                                        \
    }                                                                                                                  \
    extern "C" void orc_col2im_##S(const T* col, i64 B, i64 C, i64 H, i64 W, i64 kh, i64 kw, i64 sh, i64 sw, i64 ph,  \
                                   i64 pw, T* out, int layout) {                                                       \
        col2im<T>(col, B, C, H, W, kh, kw, sh, sw, ph, pw, out, layout);                                              \
    }                                                                                                                  \
    extern "C" void orc_gemm_naive_##S(int ta, int tb, i64 M, i64 N, i64 K, const T* A, const T* B, T* C) {           \
        gemm_naive<T>(ta, tb, M, N, K, A, B, C);                                                                      \
    }                                                                                                                  \
    extern "C" void orc_gemm_##S(int ta, int tb, i64 M, i64 N, i64 K, const T* A, const T* B, T* C) {                 \
        orc_gemm_fast<T>(ta, tb, M, N, K, A, B, C);                                                                   \
    }                                                                                                                  \
    extern "C" void orc_conv2d_fwd_##S(const T* x, const T* w, T* y, i64 B, i64 Cin, i64 H, i64 W, i64 Cout, i64 kh,  \
                                       i64 kw, i64 sh, i64 sw, i64 ph, i64 pw) {                                       \
        conv2d_fwd<T>(x, w, y, B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw);                                           \
    }                                                                                                                  \
    extern "C" void orc_conv2d_dgrad_##S(const T* g, const T* w, T* dx, i64 B, i64 Cin, i64 H, i64 W, i64 Cout,       \
                                         i64 kh, i64 kw, i64 sh, i64 sw, i64 ph, i64 pw, int mode) {                   \
        conv2d_dgrad<T>(g, w, dx, B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, mode);                                  \
    }                                                                                                                  \
    extern "C" void orc_conv2d_wgrad_##S(const T* x, const T* g, T* dw, i64 B, i64 Cin, i64 H, i64 W, i64 Cout,       \
                                         i64 kh, i64 kw, i64 sh, i64 sw, i64 ph, i64 pw, int mode) {                   \
        conv2d_wgrad<T>(x, g, dw, B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, mode);                                  \
    }                                                                                                                  \
    extern "C" void orc_binary_##S(int op, const T* a, const T* b, T* o, i64 n) { binary<T>(op, a, b, o, n); }        \
    extern "C" void orc_scalar_##S(int op, const T* a, T s, T* o, i64 n) { scalar_op<T>(op, a, s, o, n); }            \
    extern "C" void orc_unary_##S(int op, const T* a, T* o, i64 n) { unary<T>(op, a, o, n); }                         \
    extern "C" void orc_clamp_##S(const T* a, T lo, T hi, T* o, i64 n) { clamp<T>(a, lo, hi, o, n); }                 \
    extern "C" void orc_relu_bwd_##S(const T* g, const T* x, T* o, i64 n) { relu_bwd<T>(g, x, o, n); }                \
    extern "C" void orc_sigmoid_bwd_##S(const T* g, const T* s, T* o, i64 n, int literal) {                           \
        sigmoid_bwd<T>(g, s, o, n, literal);                                                                           \
    }                                                                                                                  \
    extern "C" void orc_tanh_bwd_##S(const T* g, const T* t, T* o, i64 n) { tanh_bwd<T>(g, t, o, n); }                \
    extern "C" void orc_reduce_sum_##S(const T* x, i64 outer, i64 axis, i64 inner, T* out) {                          \
        reduce_sum_axis<T>(x, outer, axis, inner, out);                                                                \
    }                                                                                                                  \
    /* mean = sum * T(1/n): cpu.rs:1193-1221 */                                                                        \
    extern "C" void orc_reduce_mean_##S(const T* x, i64 outer, i64 axis, i64 inner, T* out) {                         \
        reduce_sum_axis<T>(x, outer, axis, inner, out);                                                                \
        const T r = (T)(1.0 / (double)axis);                                                                           \
        for (i64 i = 0; i < outer * inner; ++i) out[i] = out[i] * r;                                                   \
    }                                                                                                                  \
    extern "C" void orc_reduce_max_##S(const T* x, i64 outer, i64 axis, i64 inner, T* out, i64* idx) {                \
        reduce_max_axis<T>(x, outer, axis, inner, out, idx);                                                           \
    }                                                                                                                  \
    extern "C" void orc_reduce_prod_##S(const T* x, i64 outer, i64 axis, i64 inner, T* out) {                         \
        reduce_prod_axis<T>(x, outer, axis, inner, out);                                                               \
    }                                                                                                                  \
    extern "C" void orc_reduce_min_##S(const T* x, i64 outer, i64 axis, i64 inner, T* out, i64* idx) {                \
        reduce_min_axis<T>(x, outer, axis, inner, out, idx);                                                           \
    }                                                                                                                  \
    extern "C" void orc_in_range_##S(const T* a, T lo, T hi, T* o, i64 n) { in_range<T>(a, lo, hi, o, n); }           \
    extern "C" void orc_pool2d_##S(const T* in, T* out, i64 N, i64 C, i64 H, i64 W, i64 kh, i64 kw, i64 sh, i64 sw,   \
                                   i64 ph, i64 pw, int is_max) {                                                       \
        pool2d<T>(in, out, N, C, H, W, kh, kw, sh, sw, ph, pw, is_max);                                               \
    }                                                                                                                  \
    extern "C" void orc_unpool2d_##S(const T* gout, const T* in, const T* pooled, T* gin, i64 N, i64 C, i64 H, i64 W, \
                                     i64 kh, i64 kw, i64 sh, i64 sw, i64 ph, i64 pw, int is_max) {                     \
        unpool2d<T>(gout, in, pooled, gin, N, C, H, W, kh, kw, sh, sw, ph, pw, is_max);                               \
    }                                                                                                                  \
    extern "C" void orc_softmax_axis_##S(const T* x, i64 outer, i64 axis, i64 inner, T* out) {                        \
        softmax_axis<T>(x, outer, axis, inner, out);                                                                   \
    }                                                                                                                  \
    extern "C" void orc_materialize_##S(const T* x, T* out, const i64* shape, const i64* strides, int ndim, i64 n) {  \
        materialize<T>(x, out, shape, strides, ndim, n);                                                               \
    }

ORC_INSTANTIATE(float, f32)
ORC_INSTANTIATE(double, f64)

// ---------------------------------------------------------------------------------------------
// Allocator state machine: src/backend/memory/mod.rs:225-359 (PoolBucket), src/backend/memory/cuda.rs:55-134
// (CudaMemoryPool::{allocate, deallocate, cleanup, reset}).  Integer bookkeeping only: "device blocks" are
// just records.  Timestamps are a logical counter supplied by the caller (the reference uses wall-clock ms).
// literal = 1 keeps the reference behaviour that a pool hit hands the block back under its OLD id while the
// active table recorded the NEW id (cuda.rs:61-62, 76-87), so the second release of a block is dropped.
// literal = 0 re-registers a reused block under the new id.
// ---------------------------------------------------------------------------------------------
struct OrcBlock { i64 size; uint64_t id; uint64_t ts; };
struct OrcBucket {
    i64 lo, hi; i64 cap; i64 to_evict; i64 thresh;  // thresh < 0: none
    std::vector<OrcBlock> blocks;
    i64 st_total = 0, st_evictions = 0, st_avail = 0;
};
struct OrcPool {
    std::vector<OrcBucket> buckets;
    std::vector<std::pair<uint64_t, int>> active;  // id -> bucket
    uint64_t counter = 0;
    i64 total_allocations = 0, active_allocations = 0, hits = 0, misses = 0, underflow = 0;
    i64 device_allocs = 0, device_frees = 0;
    int literal = 1;
    uint64_t clock = 0;
};

static void orc_bucket_return(OrcPool* p, OrcBucket& b, OrcBlock blk) {  // mod.rs:263-288
    const i64 cur = (i64)b.blocks.size();
    if (cur >= b.cap) {
        if (b.thresh >= 0) {  // evict_older_than, mod.rs:307-320
            const uint64_t now = p->clock;
            auto it = std::remove_if(b.blocks.begin(), b.blocks.end(),
                                     [&](const OrcBlock& x) { return (now - x.ts) > (uint64_t)b.thresh; });
            p->device_frees += (i64)(b.blocks.end() - it);
            b.blocks.erase(it, b.blocks.end());
        } else {  // evict_lru, mod.rs:291-305 : stable sort by timestamp, drop the oldest
            const i64 n = std::min<i64>(b.to_evict, (i64)b.blocks.size());
            if (n > 0) {
                std::stable_sort(b.blocks.begin(), b.blocks.end(),
                                 [](const OrcBlock& x, const OrcBlock& y) { return x.ts < y.ts; });
                b.blocks.erase(b.blocks.begin(), b.blocks.begin() + n);
                p->device_frees += n;
            }
        }
    }
    b.st_evictions += cur - (i64)b.blocks.size();
    b.st_total = (i64)b.blocks.size() + 1;
    b.st_avail = std::max<i64>(0, b.cap - ((i64)b.blocks.size() + 1));
    blk.ts = p->clock;
    b.blocks.push_back(blk);
}

extern "C" {
OrcPool* orc_pool_new(int nb, const i64* lo, const i64* hi, const i64* cap, const i64* to_evict, const i64* thresh,
                      int literal) {
    OrcPool* p = new OrcPool();
    p->literal = literal;
    for (int i = 0; i < nb; ++i) {
        OrcBucket b;
        b.lo = lo[i]; b.hi = hi[i]; b.cap = cap[i]; b.to_evict = to_evict[i]; b.thresh = thresh[i];
        b.st_avail = cap[i];
        p->buckets.push_back(b);
    }
    return p;
}
void orc_pool_delete(OrcPool* p) { delete p; }
void orc_pool_tick(OrcPool* p, uint64_t dt) { p->clock += dt; }

// returns 0 ok / -1 zero size / -2 no bucket. out: granted size, id
int orc_pool_alloc(OrcPool* p, i64 size, i64* granted, uint64_t* id_out) {  // cuda.rs:56-101
    if (size == 0) return -1;
    p->counter += 1;
    const uint64_t id = p->counter;
    int bi = -1;
    for (size_t i = 0; i < p->buckets.size(); ++i)
        if (size >= p->buckets[i].lo && size <= p->buckets[i].hi) { bi = (int)i; break; }
    if (bi < 0) return -2;
    auto set_active = [&](uint64_t k, int v) {
        for (auto& e : p->active) if (e.first == k) { e.second = v; return; }
        p->active.push_back({k, v});
    };
    set_active(id, bi);
    OrcBucket& b = p->buckets[bi];
    if (!b.blocks.empty()) {
        OrcBlock blk = b.blocks.back();
        b.blocks.pop_back();
        if (blk.size >= size) {
            p->hits += 1;
            p->active_allocations += 1;
            if (!p->literal) blk.id = id;  // fixed mode: the block now answers to the new id
            *granted = blk.size; *id_out = blk.id;
            return 0;
        }
        p->underflow += 1;
        orc_bucket_return(p, b, blk);
    }
    p->device_allocs += 1;
    set_active(id, bi);
    p->misses += 1; p->total_allocations += 1; p->active_allocations += 1;  // update_stats, cuda.rs:188-192
    *granted = size; *id_out = id;
    return 0;
}

// returns 1 if the block went back to its bucket, 0 if it was dropped (unknown id -> freed), cuda.rs:103-111
int orc_pool_free(OrcPool* p, i64 size, uint64_t id) {
    for (size_t i = 0; i < p->active.size(); ++i)
        if (p->active[i].first == id) {
            const int bi = p->active[i].second;
            p->active.erase(p->active.begin() + i);
            p->active_allocations -= 1;
            orc_bucket_return(p, p->buckets[bi], OrcBlock{size, id, 0});
            return 1;
        }
    p->device_frees += 1;
    return 0;
}
void orc_pool_cleanup(OrcPool* p) {  // cuda.rs:113-119
    for (auto& b : p->buckets) { p->device_frees += (i64)b.blocks.size(); b.blocks.clear(); }
}
void orc_pool_reset(OrcPool* p) {  // cuda.rs:125-133
    for (auto& b : p->buckets) { p->device_frees += (i64)b.blocks.size(); b.blocks.clear(); }
    p->active.clear(); p->counter = 0;
    p->total_allocations = p->active_allocations = p->hits = p->misses = p->underflow = 0;
}
// out[0..7] = total_allocations, active_allocations, hits, misses, underflow, active_table_len, device_allocs, device_frees
void orc_pool_stats(OrcPool* p, i64* out) {
    out[0] = p->total_allocations; out[1] = p->active_allocations; out[2] = p->hits; out[3] = p->misses;
    out[4] = p->underflow; out[5] = (i64)p->active.size(); out[6] = p->device_allocs; out[7] = p->device_frees;
}
// out[0..4] = pooled_count, total_allocations, total_evictions, av_allocations, max_allocations (BucketStats mod.rs:204-210)
void orc_pool_bucket_stats(OrcPool* p, int bi, i64* out) {
    const OrcBucket& b = p->buckets[bi];
    out[0] = (i64)b.blocks.size(); out[1] = b.st_total; out[2] = b.st_evictions; out[3] = b.st_avail; out[4] = b.cap;
}
}
