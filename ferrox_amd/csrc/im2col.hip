// Explicit im2col / col2im kernels: the bit-exact-layout path of the convolution
// (src/backend/storage/extensions/convolutions.rs:10-75 and 79-153).  The fast convolution entry points use an
// implicit GEMM and never build the column matrix; these kernels serve callers that want the matrix itself and
// the CPU-literal gradient mode.
//
// col2im is written as a GATHER: one thread owns one image pixel and adds the (at most kh*kw) column entries that
// map to it in ascending (ky, kx) order -- the order in which the reference's scatter loop reaches that pixel --
// so the result is race-free, deterministic and bit-identical to the CPU.
#include "common.hpp"

namespace {

struct ConvGeom {
    i64 B, C, H, W, kh, kw, sh, sw, ph, pw, oh, ow;
};

template <typename T>
__global__ __launch_bounds__(256) void im2col_kernel(const T* __restrict__ x, T* __restrict__ col, ConvGeom g) {
    const i64 n = (i64)blockIdx.x * 256 + threadIdx.x;  // column = b*oh*ow + oy*ow + ox
    const i64 row = blockIdx.y;                         // row = c*kh*kw + ky*kw + kx
    const i64 N = g.B * g.oh * g.ow;
    if (n >= N) return;
    const i64 L = g.oh * g.ow;
    const i64 b = n / L, l = n - b * L;
    const i64 oy = l / g.ow, ox = l - oy * g.ow;
    const i64 KK = g.kh * g.kw;
    const i64 c = row / KK, r = row - c * KK;
    const i64 ky = r / g.kw, kx = r - ky * g.kw;
    const i64 iy = oy * g.sh + ky - g.ph, ix = ox * g.sw + kx - g.pw;
    T v = T(0);
    if (iy >= 0 && iy < g.H && ix >= 0 && ix < g.W) v = x[((b * g.C + c) * g.H + iy) * g.W + ix];
    col[row * N + n] = v;
}

template <typename T, int LAYOUT>
__global__ __launch_bounds__(256) void col2im_kernel(const T* __restrict__ col, T* __restrict__ out, ConvGeom g) {
    const i64 idx = (i64)blockIdx.x * 256 + threadIdx.x;  // flat NCHW pixel
    const i64 total = g.B * g.C * g.H * g.W;
    if (idx >= total) return;
    const i64 xw = idx % g.W;
    i64 t = idx / g.W;
    const i64 y = t % g.H;
    t /= g.H;
    const i64 c = t % g.C;
    const i64 b = t / g.C;
    const i64 L = g.oh * g.ow, KK = g.kh * g.kw;
    const i64 Y = y + g.ph, X = xw + g.pw;  // position in the padded image
    T acc = T(0);
    for (i64 ky = 0; ky < g.kh; ++ky) {
        const i64 ty = Y - ky;
        if (ty < 0) break;
        if (ty % g.sh != 0) continue;
        const i64 cy = ty / g.sh;
        if (cy >= g.oh) continue;
        for (i64 kx = 0; kx < g.kw; ++kx) {
            const i64 tx = X - kx;
            if (tx < 0) break;
            if (tx % g.sw != 0) continue;
            const i64 cx = tx / g.sw;
            if (cx >= g.ow) continue;
            i64 ci;
            if (LAYOUT == 1)
                ci = b * (g.C * KK * L) + c * (KK * L) + ky * (g.kw * L) + kx * L + cy * g.ow + cx;
            else
                ci = (c * KK + ky * g.kw + kx) * (g.B * L) + b * L + cy * g.ow + cx;
            acc = acc + col[ci];
        }
    }
    out[idx] = acc;
}

int make_geom(ConvGeom& g, i64 B, i64 C, i64 H, i64 W, i64 kh, i64 kw, i64 sh, i64 sw, i64 ph, i64 pw, const char* what) {
    FX_REQUIRE(B > 0 && C > 0 && H > 0 && W > 0 && kh > 0 && kw > 0 && sh > 0 && sw > 0 && ph >= 0 && pw >= 0,
               "%s: non-positive dimension", what);
    FX_REQUIRE(H + 2 * ph >= kh && W + 2 * pw >= kw, "%s: kernel larger than padded input", what);
    g = ConvGeom{B, C, H, W, kh, kw, sh, sw, ph, pw, (H + 2 * ph - kh) / sh + 1, (W + 2 * pw - kw) / sw + 1};
    return FX_OK;
}

// ---- 32-bit variants (every tensor below 2^31 elements): multiply-shift divisions, no 64-bit index arithmetic ------
// n / d for 32-bit n by multiply-shift (d fixed per launch)
struct U32Div {
    uint32_t d, m, s;
    __device__ __forceinline__ uint32_t div(uint32_t n) const { return (uint32_t)(((uint64_t)__umulhi(n, m) + n) >> s); }
};
U32Div make_div(uint32_t d) {
    U32Div r;
    r.d = d;
    r.s = 0;
    while ((1ull << r.s) < d) ++r.s;
    r.m = (uint32_t)((((1ull << 32) * ((1ull << r.s) - d)) / d) + 1);
    return r;
}
struct Geom32 {
    int B, C, H, W, kh, kw, sh, sw, ph, pw, oh, ow;
    U32Div div_L, div_ow, div_KK, div_kw, div_W, div_H, div_C, div_sh, div_sw;
};

// One thread writes V consecutive columns of one row of the column matrix (one 16-byte store when V > 1); the row's
// (c, ky, kx) is block-uniform (blockIdx.y), the first column is decoded once and the rest follow by increments.
template <typename T, int V>
__global__ __launch_bounds__(256) void im2col32_kernel(const T* __restrict__ x, T* __restrict__ col, Geom32 g, uint32_t N) {
    typedef T vec_t __attribute__((ext_vector_type(V)));
    const uint32_t n0 = (blockIdx.x * 256u + threadIdx.x) * V;
    if (n0 >= N) return;
    const uint32_t row = blockIdx.y;
    const uint32_t c = g.div_KK.div(row), r = row - c * (uint32_t)(g.kh * g.kw);
    const uint32_t ky = g.div_kw.div(r), kx = r - ky * (uint32_t)g.kw;
    const uint32_t L = (uint32_t)(g.oh * g.ow);
    uint32_t b = g.div_L.div(n0), l = n0 - b * L;
    uint32_t oy = g.div_ow.div(l), ox = l - oy * (uint32_t)g.ow;
    vec_t v;
    if (ox + V <= (uint32_t)g.ow && n0 + V <= N) {
        // the V columns lie in one output row: one source row, consecutive taps; clamped loads and selects, no branches
        const int iy = (int)(oy * g.sh + ky) - g.ph, ix0 = (int)(ox * g.sw + kx) - g.pw;
        const bool row_ok = iy >= 0 && iy < g.H;
        const T* src = x + ((b * (uint32_t)g.C + c) * (uint32_t)g.H + (uint32_t)(row_ok ? iy : 0)) * (uint32_t)g.W;
#pragma unroll
        for (int u = 0; u < V; ++u) {
            const int ix = ix0 + u * g.sw;
            const bool ok = row_ok && ix >= 0 && ix < g.W;
            const T e = src[ok ? ix : 0];
            v[u] = ok ? e : T(0);
        }
        *reinterpret_cast<vec_t*>(col + (i64)row * N + n0) = v;
        return;
    }
#pragma unroll
    for (int u = 0; u < V; ++u) {
        const int iy = (int)(oy * g.sh + ky) - g.ph, ix = (int)(ox * g.sw + kx) - g.pw;
        T e = T(0);
        if (n0 + u < N && iy >= 0 && iy < g.H && ix >= 0 && ix < g.W) e = x[((i64)(b * g.C + c) * g.H + iy) * g.W + ix];
        v[u] = e;
        if (++ox == (uint32_t)g.ow) {
            ox = 0;
            if (++oy == (uint32_t)g.oh) { oy = 0; ++b; }
        }
    }
    *reinterpret_cast<vec_t*>(col + (i64)row * N + n0) = v;
}

// 3 x 3 windows at horizontal stride SW (1 or 2): one thread writes V consecutive columns of ALL nine rows of one input
// channel.  Per window row it loads the (V - 1) SW + 3 input values under its columns once (clamped loads and selects) and
// stores the three shifted vectors, so the index arithmetic and the reads are shared by nine outputs.  The V columns lie in
// one output row (ow % V == 0); blockIdx.y is the channel.
template <typename T, int V, int SW>
__global__ __launch_bounds__(256) void im2col32_w3_kernel(const T* __restrict__ x, T* __restrict__ col, Geom32 g, uint32_t N) {
    typedef T vec_t __attribute__((ext_vector_type(V)));
    const uint32_t n0 = (blockIdx.x * 256u + threadIdx.x) * V;
    if (n0 >= N) return;
    const uint32_t c = blockIdx.y;
    const uint32_t L = (uint32_t)(g.oh * g.ow);
    const uint32_t b = g.div_L.div(n0), l = n0 - b * L;
    const uint32_t oy = g.div_ow.div(l), ox = l - oy * (uint32_t)g.ow;
    const int ix0 = (int)ox * SW - g.pw;
    const T* plane = x + (b * (uint32_t)g.C + c) * (uint32_t)(g.H * g.W);
    T* dst = col + (i64)(c * 9u) * N + n0;
#pragma unroll
    for (int ky = 0; ky < 3; ++ky) {
        const int iy = (int)(oy * g.sh) + ky - g.ph;
        const bool row_ok = iy >= 0 && iy < g.H;
        const T* src = plane + (uint32_t)(row_ok ? iy : 0) * (uint32_t)g.W;
        constexpr int NB = (V - 1) * SW + 3;
        T buf[NB];
        if (ix0 >= 0 && ix0 + NB <= g.W) {
            // all NB values lie inside the row: V-wide loads at element alignment (the hardware takes unaligned vectors)
            typedef T vecu_t __attribute__((ext_vector_type(V), aligned(sizeof(T))));
            constexpr int NV = NB / V, REST = NB - NV * V;
#pragma unroll
            for (int q = 0; q < NV; ++q) {
                const vecu_t v = *reinterpret_cast<const vecu_t*>(src + ix0 + q * V);
#pragma unroll
                for (int e = 0; e < V; ++e) buf[q * V + e] = row_ok ? v[e] : T(0);
            }
#pragma unroll
            for (int e = 0; e < REST; ++e) {
                const T v = src[ix0 + NV * V + e];
                buf[NV * V + e] = row_ok ? v : T(0);
            }
        } else {
#pragma unroll
            for (int j = 0; j < NB; ++j) {
                const int ix = ix0 + j;
                const bool ok = row_ok && ix >= 0 && ix < g.W;
                const T e = src[ok ? ix : 0];
                buf[j] = ok ? e : T(0);
            }
        }
#pragma unroll
        for (int kx = 0; kx < 3; ++kx) {
            vec_t v;
#pragma unroll
            for (int u = 0; u < V; ++u) v[u] = buf[u * SW + kx];
            *reinterpret_cast<vec_t*>(dst + (i64)(ky * 3 + kx) * N) = v;
        }
    }
}

// The gather of col2im_kernel with 32-bit indices: the taps that reach a pixel are ky = (Y mod sh) + j*sh, visited in
// ascending order with cy = Y/sh - j (the same order and operands as the 64-bit kernel, so the same bits).
template <typename T, int LAYOUT>
__global__ __launch_bounds__(256) void col2im32_kernel(const T* __restrict__ col, T* __restrict__ out, Geom32 g, uint32_t total) {
    const uint32_t idx = blockIdx.x * 256u + threadIdx.x;
    if (idx >= total) return;
    uint32_t t = g.div_W.div(idx);
    const uint32_t xw = idx - t * (uint32_t)g.W;
    const uint32_t t2 = g.div_H.div(t), y = t - t2 * (uint32_t)g.H;
    const uint32_t b = g.div_C.div(t2), c = t2 - b * (uint32_t)g.C;
    const uint32_t L = (uint32_t)(g.oh * g.ow), KK = (uint32_t)(g.kh * g.kw);
    const uint32_t Y = y + (uint32_t)g.ph, X = xw + (uint32_t)g.pw;
    const uint32_t qy = g.div_sh.div(Y), ry = Y - qy * (uint32_t)g.sh;
    const uint32_t qx = g.div_sw.div(X), rx = X - qx * (uint32_t)g.sw;
    const i64 base = LAYOUT == 1 ? (i64)(b * g.C + c) * KK * L : (i64)c * KK * ((i64)g.B * L) + (i64)b * L;
    const i64 tap_stride = LAYOUT == 1 ? (i64)L : (i64)g.B * L;
    T acc = T(0);
    int cy = (int)qy;
    for (int ky = (int)ry; ky < g.kh && cy >= 0; ky += g.sh, --cy) {
        if (cy >= g.oh) continue;
        int cx = (int)qx;
        for (int kx = (int)rx; kx < g.kw && cx >= 0; kx += g.sw, --cx) {
            if (cx >= g.ow) continue;
            acc = acc + col[base + (i64)(ky * g.kw + kx) * tap_stride + cy * g.ow + cx];
        }
    }
    out[idx] = acc;
}

// Compile-time window and strides: the taps that reach a pixel are ky = (Y mod SH) + j SH with cy = Y / SH - j, j below
// ceil(KH / SH), and likewise along x -- the loop of the kernel above, unrolled, every tap one clamped load and a select
// (same taps in the same order, so the same bits; a tap outside the window or the column matrix adds nothing).
template <typename T, int LAYOUT, int KH, int KW, int SH, int SW>
__global__ __launch_bounds__(256) void col2im32_fixed_kernel(const T* __restrict__ col, T* __restrict__ out, Geom32 g, uint32_t total) {
    const uint32_t idx = blockIdx.x * 256u + threadIdx.x;
    if (idx >= total) return;
    uint32_t t = g.div_W.div(idx);
    const uint32_t xw = idx - t * (uint32_t)g.W;
    const uint32_t t2 = g.div_H.div(t), y = t - t2 * (uint32_t)g.H;
    const uint32_t b = g.div_C.div(t2), c = t2 - b * (uint32_t)g.C;
    const uint32_t L = (uint32_t)(g.oh * g.ow);
    constexpr uint32_t KK = KH * KW;
    constexpr int NJH = (KH + SH - 1) / SH, NJW = (KW + SW - 1) / SW;
    const int Y = (int)y + g.ph, X = (int)xw + g.pw;
    const int qy = Y / SH, ry = Y - qy * SH, qx = X / SW, rx = X - qx * SW;
    const i64 tap_stride = LAYOUT == 1 ? (i64)L : (i64)g.B * L;
    const T* base = col + (LAYOUT == 1 ? (i64)(b * g.C + c) * KK * L : (i64)c * KK * ((i64)g.B * L) + (i64)b * L);
    T acc = T(0);
#pragma unroll
    for (int jy = 0; jy < NJH; ++jy) {
        const int ky = ry + jy * SH, cy = qy - jy;
        const bool row_ok = ky < KH && cy >= 0 && cy < g.oh;
#pragma unroll
        for (int jx = 0; jx < NJW; ++jx) {
            const int kx = rx + jx * SW, cx = qx - jx;
            const bool ok = row_ok && kx < KW && cx >= 0 && cx < g.ow;
            const T v = base[(ok ? (i64)(ky * KW + kx) * tap_stride + cy * g.ow + cx : (i64)0)];
            acc = ok ? acc + v : acc;
        }
    }
    out[idx] = acc;
}

bool geom32(Geom32& q, const ConvGeom& g) {
    const i64 N = g.B * g.oh * g.ow;
    const i64 lim = 0x7fffffff;
    if (g.B * g.C * g.H * g.W > lim || N > lim - 4 || g.H + 2 * g.ph > lim || g.W + 2 * g.pw > lim) return false;
    q.B = (int)g.B; q.C = (int)g.C; q.H = (int)g.H; q.W = (int)g.W; q.kh = (int)g.kh; q.kw = (int)g.kw;
    q.sh = (int)g.sh; q.sw = (int)g.sw; q.ph = (int)g.ph; q.pw = (int)g.pw; q.oh = (int)g.oh; q.ow = (int)g.ow;
    q.div_L = make_div((uint32_t)(g.oh * g.ow)); q.div_ow = make_div((uint32_t)g.ow);
    q.div_KK = make_div((uint32_t)(g.kh * g.kw)); q.div_kw = make_div((uint32_t)g.kw);
    q.div_W = make_div((uint32_t)g.W); q.div_H = make_div((uint32_t)g.H); q.div_C = make_div((uint32_t)g.C);
    q.div_sh = make_div((uint32_t)g.sh); q.div_sw = make_div((uint32_t)g.sw);
    return true;
}

template <typename T>
int im2col(fx_ctx* c, const T* x, T* col, i64 B, i64 C, i64 H, i64 W, i64 kh, i64 kw, i64 sh, i64 sw, i64 ph, i64 pw) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(x && col, "fx_im2col: null pointer");
    ConvGeom g;
    if (int rc = make_geom(g, B, C, H, W, kh, kw, sh, sw, ph, pw, "fx_im2col")) return rc;
    const i64 N = B * g.oh * g.ow, rows = C * kh * kw;
    FX_REQUIRE(rows <= 65535, "fx_im2col: C*kh*kw = %lld exceeds 65535", (long long)rows);
    FX_REQUIRE(fx::ceil_div(N, 256) <= 0x7fffffff, "fx_im2col: too many columns");
    Geom32 q;
    if (geom32(q, g)) {
        constexpr int V = 16 / (int)sizeof(T);
        if (kh == 3 && kw == 3 && sw == 1 && g.ow % V == 0 && fx::aligned16(col))
            im2col32_w3_kernel<T, V, 1><<<dim3((unsigned)fx::ceil_div(N / V, 256), (unsigned)C), dim3(256), 0, c->stream>>>(x, col, q, (uint32_t)N);
        else if (kh == 3 && kw == 3 && sw == 2 && g.ow % V == 0 && fx::aligned16(col))
            im2col32_w3_kernel<T, V, 2><<<dim3((unsigned)fx::ceil_div(N / V, 256), (unsigned)C), dim3(256), 0, c->stream>>>(x, col, q, (uint32_t)N);
        else if (N % V == 0 && fx::aligned16(col))
            im2col32_kernel<T, V><<<dim3((unsigned)fx::ceil_div(N / V, 256), (unsigned)rows), dim3(256), 0, c->stream>>>(x, col, q, (uint32_t)N);
        else
            im2col32_kernel<T, 1><<<dim3((unsigned)fx::ceil_div(N, 256), (unsigned)rows), dim3(256), 0, c->stream>>>(x, col, q, (uint32_t)N);
        FX_LAUNCH_CHECK();
        return FX_OK;
    }
    im2col_kernel<T><<<dim3((unsigned)fx::ceil_div(N, 256), (unsigned)rows), dim3(256), 0, c->stream>>>(x, col, g);
    FX_LAUNCH_CHECK();
    return FX_OK;
}

template <typename T>
int col2im(fx_ctx* c, const T* col, T* out, i64 B, i64 C, i64 H, i64 W, i64 kh, i64 kw, i64 sh, i64 sw, i64 ph, i64 pw,
           int layout) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(col && out, "fx_col2im: null pointer");
    FX_REQUIRE(layout == 0 || layout == 1, "fx_col2im: layout must be 0 or 1");
    ConvGeom g;
    if (int rc = make_geom(g, B, C, H, W, kh, kw, sh, sw, ph, pw, "fx_col2im")) return rc;
    const i64 total = B * C * H * W;
    FX_REQUIRE(fx::ceil_div(total, 256) <= 0x7fffffff, "fx_col2im: too many pixels");
    const dim3 grid((unsigned)fx::ceil_div(total, 256)), block(256);
    Geom32 q;
    if (geom32(q, g)) {
        const bool k3 = kh == 3 && kw == 3, s1 = k3 && sh == 1 && sw == 1, s2 = k3 && sh == 2 && sw == 2;
        if (s1 && layout == 1) col2im32_fixed_kernel<T, 1, 3, 3, 1, 1><<<grid, block, 0, c->stream>>>(col, out, q, (uint32_t)total);
        else if (s1) col2im32_fixed_kernel<T, 0, 3, 3, 1, 1><<<grid, block, 0, c->stream>>>(col, out, q, (uint32_t)total);
        else if (s2 && layout == 1) col2im32_fixed_kernel<T, 1, 3, 3, 2, 2><<<grid, block, 0, c->stream>>>(col, out, q, (uint32_t)total);
        else if (s2) col2im32_fixed_kernel<T, 0, 3, 3, 2, 2><<<grid, block, 0, c->stream>>>(col, out, q, (uint32_t)total);
        else if (layout == 1) col2im32_kernel<T, 1><<<grid, block, 0, c->stream>>>(col, out, q, (uint32_t)total);
        else col2im32_kernel<T, 0><<<grid, block, 0, c->stream>>>(col, out, q, (uint32_t)total);
        FX_LAUNCH_CHECK();
        return FX_OK;
    }
    if (layout == 1) col2im_kernel<T, 1><<<grid, block, 0, c->stream>>>(col, out, g);
    else col2im_kernel<T, 0><<<grid, block, 0, c->stream>>>(col, out, g);
    FX_LAUNCH_CHECK();
    return FX_OK;
}

}  // namespace

namespace fx {
// used by the literal-mode data gradient in igemm.hip
int col2im_f32(fx_ctx* c, const float* col, float* out, i64 B, i64 C, i64 H, i64 W, i64 kh, i64 kw, i64 sh, i64 sw, i64 ph, i64 pw, int layout) {
    return col2im<float>(c, col, out, B, C, H, W, kh, kw, sh, sw, ph, pw, layout);
}
int col2im_f64(fx_ctx* c, const double* col, double* out, i64 B, i64 C, i64 H, i64 W, i64 kh, i64 kw, i64 sh, i64 sw, i64 ph, i64 pw, int layout) {
    return col2im<double>(c, col, out, B, C, H, W, kh, kw, sh, sw, ph, pw, layout);
}
}  // namespace fx

#define FX_DEFINE_IM2COL(T, S)                                                                                         \
    extern "C" int fx_im2col_##S(fx_ctx* c, const T* x, T* col, int64_t B, int64_t C, int64_t H, int64_t W, int64_t kh, \
                                 int64_t kw, int64_t sh, int64_t sw, int64_t ph, int64_t pw) {                         \
        return im2col<T>(c, x, col, B, C, H, W, kh, kw, sh, sw, ph, pw);                                               \
    }                                                                                                                  \
    extern "C" int fx_col2im_##S(fx_ctx* c, const T* col, T* out, int64_t B, int64_t C, int64_t H, int64_t W,          \
                                 int64_t kh, int64_t kw, int64_t sh, int64_t sw, int64_t ph, int64_t pw, int layout) { \
        return col2im<T>(c, col, out, B, C, H, W, kh, kw, sh, sw, ph, pw, layout);                                     \
    }

FX_DEFINE_IM2COL(float, f32)
FX_DEFINE_IM2COL(double, f64)
