// Max / average pooling and their gradients ("unpooling"), NCHW, as the reference's CPU backend computes them
// (src/backend/storage/extensions/pooling.rs:154-229, 339-418; its CUDA twins are kernels/convolutions.cu:671-1222).
// The 1-D variants ([N, C, L], pooling.rs:231-287, 420-488) are the same kernels with H = 1 and a 1 x k window.
//   pool    out[n,c,oy,ox]: window rows ky, columns kx ascending over the in-bounds part of
//           [oy*s - p, +k) x [ox*s - p, +k); max starts from the lowest finite T and takes strictly greater values;
//           avg divides the running sum by the number of in-bounds elements (0 when there is none).
//   unpool  grad_in[n,c,y,x] = sum over the windows (oy, ox ascending) that contain (y, x) of
//           max: grad_out where |in - pooled| < 1e-8;   avg: grad_out * T(1.0f / float(kh*kw)).
// Same operations in the same order as the CPU loops -> bit-identical (this file is built without contraction).
#include <algorithm>

#include "common.hpp"

namespace {

// n / d for 32-bit n by multiply-shift (d fixed per launch)
struct U32Div {
    uint32_t d, m, s;
    __device__ __forceinline__ uint32_t div(uint32_t n) const { return (uint32_t)(((uint64_t)__umulhi(n, m) + n) >> s); }
};
static U32Div make_div(uint32_t d) {
    U32Div r;
    r.d = d;
    r.s = 0;
    while ((1ull << r.s) < d) ++r.s;
    r.m = (uint32_t)((((1ull << 32) * ((1ull << r.s) - d)) / d) + 1);
    return r;
}

struct PoolShape {
    int C, H, W, oh, ow, kh, kw, sh, sw, ph, pw;
    U32Div div_W, div_H, div_ow, div_oh, div_sh, div_sw;
};

template <typename T> __device__ __forceinline__ T lowest_finite();
template <> __device__ __forceinline__ float lowest_finite<float>() { return -3.402823466e+38f; }
template <> __device__ __forceinline__ double lowest_finite<double>() { return -1.7976931348623157e+308; }

// One thread per output element; tensors below 2^31 elements (checked on the host) so index arithmetic is 32-bit.
template <typename T, bool IS_MAX>
__global__ __launch_bounds__(256) void pool2d_kernel(const T* __restrict__ in, T* __restrict__ out, PoolShape s, uint32_t n_out) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= n_out) return;
    uint32_t t = s.div_ow.div(i);
    const int ox = (int)(i - t * s.ow);
    const uint32_t plane = s.div_oh.div(t);
    const int oy = (int)(t - plane * s.oh);
    const T* p = in + (i64)plane * s.H * s.W;
    const int y0 = oy * s.sh - s.ph, x0 = ox * s.sw - s.pw;
    T acc = IS_MAX ? lowest_finite<T>() : T(0);
    int count = 0;
    for (int ky = 0; ky < s.kh; ++ky) {
        const int y = y0 + ky;
        if (y < 0 || y >= s.H) continue;
        for (int kx = 0; kx < s.kw; ++kx) {
            const int x = x0 + kx;
            if (x < 0 || x >= s.W) continue;
            const T v = p[y * s.W + x];
            if (IS_MAX) { if (v > acc) acc = v; }
            else { acc = acc + v; ++count; }
        }
    }
    if (!IS_MAX) acc = count > 0 ? acc / (T)count : T(0);
    out[i] = acc;
}

// The common non-overlapping 2x2 / stride 2 / no padding window on even W: a lane reads its two columns as one
// 8- or 16-byte vector, so a wave reads whole contiguous lines.  Same visiting order (ky, kx) as the general kernel.
template <typename T, bool IS_MAX>
__global__ __launch_bounds__(256) void pool2d_2x2_kernel(const T* __restrict__ in, T* __restrict__ out, PoolShape s, uint32_t n_out) {
    typedef T vec2 __attribute__((ext_vector_type(2)));
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= n_out) return;
    uint32_t t = s.div_ow.div(i);
    const int ox = (int)(i - t * s.ow);
    const uint32_t plane = s.div_oh.div(t);
    const int oy = (int)(t - plane * s.oh);
    const T* p = in + ((i64)plane * s.H + 2 * oy) * s.W + 2 * ox;
    const vec2 r0 = *reinterpret_cast<const vec2*>(p), r1 = *reinterpret_cast<const vec2*>(p + s.W);
    T acc;
    if (IS_MAX) {
        acc = lowest_finite<T>();
        if (r0.x > acc) acc = r0.x;
        if (r0.y > acc) acc = r0.y;
        if (r1.x > acc) acc = r1.x;
        if (r1.y > acc) acc = r1.y;
    } else {
        acc = T(0);
        acc = acc + r0.x;
        acc = acc + r0.y;
        acc = acc + r1.x;
        acc = acc + r1.y;
        acc = acc / T(4);
    }
    out[i] = acc;
}

template <typename T, bool IS_MAX>
__global__ __launch_bounds__(256) void unpool2d_kernel(const T* __restrict__ gout, const T* __restrict__ in, const T* __restrict__ pooled,
                                                       T* __restrict__ gin, PoolShape s, uint32_t n_in, T scale, T eps) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= n_in) return;
    uint32_t t = s.div_W.div(i);
    const int x = (int)(i - t * s.W);
    const uint32_t plane = s.div_H.div(t);
    const int y = (int)(t - plane * s.H);
    const T* go = gout + (i64)plane * s.oh * s.ow;
    const T* po = pooled + (i64)plane * s.oh * s.ow;
    const T orig = IS_MAX ? in[i] : T(0);
    // windows containing (y, x): oy*sh - ph <= y < oy*sh - ph + kh
    int oy_lo = y + s.ph - s.kh + 1;
    oy_lo = oy_lo <= 0 ? 0 : (int)s.div_sh.div((uint32_t)(oy_lo + s.sh - 1));
    int oy_hi = (int)s.div_sh.div((uint32_t)(y + s.ph));
    if (oy_hi > s.oh - 1) oy_hi = s.oh - 1;
    int ox_lo = x + s.pw - s.kw + 1;
    ox_lo = ox_lo <= 0 ? 0 : (int)s.div_sw.div((uint32_t)(ox_lo + s.sw - 1));
    int ox_hi = (int)s.div_sw.div((uint32_t)(x + s.pw));
    if (ox_hi > s.ow - 1) ox_hi = s.ow - 1;
    T acc = T(0);
    for (int oy = oy_lo; oy <= oy_hi; ++oy)
        for (int ox = ox_lo; ox <= ox_hi; ++ox) {
            const T g = go[oy * s.ow + ox];
            if (IS_MAX) {
                const T pv = po[oy * s.ow + ox];
                const T diff = orig > pv ? orig - pv : pv - orig;
                if (diff < eps) acc = acc + g;
            } else {
                acc = acc + g * scale;
            }
        }
    gin[i] = acc;
}

// Gradient of the non-overlapping 2x2 / stride 2 / no padding window on even H and W: every input element lies in
// exactly one window, so one thread owns a window and writes its four gradients as two vectors.
template <typename T, bool IS_MAX>
__global__ __launch_bounds__(256) void unpool2d_2x2_kernel(const T* __restrict__ gout, const T* __restrict__ in, const T* __restrict__ pooled,
                                                           T* __restrict__ gin, PoolShape s, uint32_t n_out, T scale, T eps) {
    typedef T vec2 __attribute__((ext_vector_type(2)));
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= n_out) return;
    uint32_t t = s.div_ow.div(i);
    const int ox = (int)(i - t * s.ow);
    const uint32_t plane = s.div_oh.div(t);
    const int oy = (int)(t - plane * s.oh);
    const i64 base = ((i64)plane * s.H + 2 * oy) * s.W + 2 * ox;
    const T g = gout[i];
    vec2 o0, o1;
    if (IS_MAX) {
        const T pv = pooled[i];
        const vec2 r0 = *reinterpret_cast<const vec2*>(in + base), r1 = *reinterpret_cast<const vec2*>(in + base + s.W);
        auto pick = [&](T orig) {
            const T diff = orig > pv ? orig - pv : pv - orig;
            return diff < eps ? T(0) + g : T(0);
        };
        o0.x = pick(r0.x); o0.y = pick(r0.y); o1.x = pick(r1.x); o1.y = pick(r1.y);
    } else {
        const T v = T(0) + g * scale;
        o0.x = o0.y = o1.x = o1.y = v;
    }
    *reinterpret_cast<vec2*>(gin + base) = o0;
    *reinterpret_cast<vec2*>(gin + base + s.W) = o1;
}

template <typename T>
int check_pool(PoolShape& s, i64 N, i64 C, i64 H, i64 W, i64 kh, i64 kw, i64 sh, i64 sw, i64 ph, i64 pw, const char* what) {
    FX_REQUIRE(N > 0 && C > 0 && H > 0 && W > 0 && kh > 0 && kw > 0 && sh > 0 && sw > 0 && ph >= 0 && pw >= 0, "%s: non-positive dimension", what);
    FX_REQUIRE(H + 2 * ph >= kh && W + 2 * pw >= kw, "%s: window larger than padded input", what);
    FX_REQUIRE(H < (1 << 24) && W < (1 << 24) && kh < 32768 && kw < 32768 && ph < 32768 && pw < 32768 && C < (1ll << 31), "%s: dimension too large", what);
    s = PoolShape{(int)C, (int)H, (int)W, (int)((H + 2 * ph - kh) / sh + 1), (int)((W + 2 * pw - kw) / sw + 1),
                  (int)kh, (int)kw, (int)sh, (int)sw, (int)ph, (int)pw, {}, {}, {}, {}, {}, {}};
    s.div_W = make_div((uint32_t)W);
    s.div_H = make_div((uint32_t)H);
    s.div_ow = make_div((uint32_t)s.ow);
    s.div_oh = make_div((uint32_t)s.oh);
    s.div_sh = make_div((uint32_t)sh);
    s.div_sw = make_div((uint32_t)sw);
    if (std::max(H * W, (i64)s.oh * s.ow) >= (1ll << 31)) {
        fx::set_error("%s: planes of 2^31 elements or more are not supported by this build", what);
        return FX_ERR_UNSUPPORTED;
    }
    return FX_OK;
}

// The kernels number the elements of one launch with 32 bits.  Planes (image x channel) are independent, so a larger
// tensor runs as several launches over ranges of planes; returns how many planes one launch may take.
inline i64 planes_per_launch(const PoolShape& s, i64 planes) {
    const i64 per = std::max((i64)s.H * s.W, (i64)s.oh * s.ow);
    return std::min<i64>(planes, (((i64)1 << 31) - 1) / per);
}

template <typename T, bool IS_MAX>
int pool2d(fx_ctx* c, const T* in, T* out, i64 N, i64 C, i64 H, i64 W, i64 kh, i64 kw, i64 sh, i64 sw, i64 ph, i64 pw, const char* what) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(in && out, "%s: null pointer", what);
    PoolShape s;
    if (int rc = check_pool<T>(s, N, C, H, W, kh, kw, sh, sw, ph, pw, what)) return rc;
    const i64 planes = N * C, ppl = planes_per_launch(s, planes);
    if (planes > ppl) {
        for (i64 p0 = 0; p0 < planes; p0 += ppl)
            if (int rc = pool2d<T, IS_MAX>(c, in + p0 * H * W, out + p0 * s.oh * s.ow, std::min(ppl, planes - p0), 1, H, W, kh, kw, sh, sw, ph, pw, what))
                return rc;
        return FX_OK;
    }
    const i64 n_out = N * C * s.oh * s.ow, blocks = fx::ceil_div(n_out, (i64)256);
    if (n_out == 0) return FX_OK;
    if (kh == 2 && kw == 2 && sh == 2 && sw == 2 && ph == 0 && pw == 0 && W % 2 == 0 && ((uintptr_t)in % (2 * sizeof(T))) == 0)
        pool2d_2x2_kernel<T, IS_MAX><<<dim3((unsigned)blocks), dim3(256), 0, c->stream>>>(in, out, s, (uint32_t)n_out);
    else
        pool2d_kernel<T, IS_MAX><<<dim3((unsigned)blocks), dim3(256), 0, c->stream>>>(in, out, s, (uint32_t)n_out);
    FX_LAUNCH_CHECK();
    return FX_OK;
}

template <typename T, bool IS_MAX>
int unpool2d(fx_ctx* c, const T* gout, const T* in, const T* pooled, T* gin, i64 N, i64 C, i64 H, i64 W, i64 kh, i64 kw, i64 sh,
             i64 sw, i64 ph, i64 pw, const char* what) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(gout && gin && (!IS_MAX || (in && pooled)), "%s: null pointer", what);
    PoolShape s;
    if (int rc = check_pool<T>(s, N, C, H, W, kh, kw, sh, sw, ph, pw, what)) return rc;
    const i64 planes = N * C, ppl = planes_per_launch(s, planes);
    if (planes > ppl) {
        for (i64 p0 = 0; p0 < planes; p0 += ppl) {
            const i64 oi = p0 * H * W, oo = p0 * s.oh * s.ow;
            if (int rc = unpool2d<T, IS_MAX>(c, gout + oo, in ? in + oi : nullptr, pooled ? pooled + oo : nullptr, gin + oi,
                                             std::min(ppl, planes - p0), 1, H, W, kh, kw, sh, sw, ph, pw, what))
                return rc;
        }
        return FX_OK;
    }
    const i64 n_in = N * C * H * W, blocks = fx::ceil_div(n_in, (i64)256);
    const float area = (float)(kh * kw);  // kernel_area is an f32 in the reference, for f64 tensors too (pooling.rs:361, 138)
    const T scale = (T)(1.0f / area);
    const bool al = ((uintptr_t)gin % (2 * sizeof(T))) == 0 && (!IS_MAX || ((uintptr_t)in % (2 * sizeof(T))) == 0);
    if (kh == 2 && kw == 2 && sh == 2 && sw == 2 && ph == 0 && pw == 0 && W % 2 == 0 && H % 2 == 0 && al) {
        const i64 n_out = n_in / 4;
        unpool2d_2x2_kernel<T, IS_MAX><<<dim3((unsigned)fx::ceil_div(n_out, (i64)256)), dim3(256), 0, c->stream>>>(
            gout, in, pooled, gin, s, (uint32_t)n_out, scale, (T)1e-8f);
    } else {
        unpool2d_kernel<T, IS_MAX><<<dim3((unsigned)blocks), dim3(256), 0, c->stream>>>(gout, in, pooled, gin, s, (uint32_t)n_in, scale, (T)1e-8f);
    }
    FX_LAUNCH_CHECK();
    return FX_OK;
}

}  // namespace

#define FX_POOL_ARGS int64_t N, int64_t C, int64_t H, int64_t W, int64_t kh, int64_t kw, int64_t sh, int64_t sw, int64_t ph, int64_t pw
#define FX_POOL_PASS N, C, H, W, kh, kw, sh, sw, ph, pw
#define FX_DEFINE_POOL(T, S)                                                                                           \
    extern "C" int fx_maxpool2d_##S(fx_ctx* c, const T* in, T* out, FX_POOL_ARGS) {                                    \
        return pool2d<T, true>(c, in, out, FX_POOL_PASS, "fx_maxpool2d");                                              \
    }                                                                                                                  \
    extern "C" int fx_avgpool2d_##S(fx_ctx* c, const T* in, T* out, FX_POOL_ARGS) {                                    \
        return pool2d<T, false>(c, in, out, FX_POOL_PASS, "fx_avgpool2d");                                             \
    }                                                                                                                  \
    extern "C" int fx_max_unpool2d_##S(fx_ctx* c, const T* grad_out, const T* in, const T* pooled, T* grad_in, FX_POOL_ARGS) { \
        return unpool2d<T, true>(c, grad_out, in, pooled, grad_in, FX_POOL_PASS, "fx_max_unpool2d");                   \
    }                                                                                                                  \
    extern "C" int fx_avg_unpool2d_##S(fx_ctx* c, const T* grad_out, T* grad_in, FX_POOL_ARGS) {                       \
        return unpool2d<T, false>(c, grad_out, nullptr, nullptr, grad_in, FX_POOL_PASS, "fx_avg_unpool2d");            \
    }

FX_DEFINE_POOL(float, f32)
FX_DEFINE_POOL(double, f64)
