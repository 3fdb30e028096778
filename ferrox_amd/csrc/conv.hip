// Conv2d forward, data-gradient and weight-gradient as implicit GEMMs on the MFMA pipes.
//
// The reference CPU backend builds an explicit im2col matrix (925 MB for N=128,C=64,56x56,k3), multiplies, and
// transposes or scatters the result (src/backend/storage/extensions/convolutions.rs:218-338); its CUDA backend
// uses direct kernels (kernels/convolutions.cu).  Here the three passes are GEMMs whose operand loaders do the
// im2col / col2im index arithmetic while filling LDS, so HBM traffic stays at the tensors themselves:
//   fwd  : y[b,oc,l]   = sum_{c,ky,kx} w[oc,(c,ky,kx)] * x[b,c,oy*s+ky-p,ox*s+kx-p]   M=Cout N=B*oh*ow K=Cin*kh*kw
//   dgrad: dx[b,c,p]   = sum_{oc,ky,kx} wt[c,(oc,ky,kx)] * g[b,oc,(y+p-ky)/s,(x+p-kx)/s] M=Cin  N=B*H*W   K=Cout*kh*kw
//          (gather form of col2im: one accumulator owns each input pixel -> race-free and deterministic)
//   wgrad: dw[oc,(c,ky,kx)] = sum_{b,l} g[b,oc,l] * x[b,c,...]                         M=Cout N=Cin*kh*kw K=B*oh*ow
//          (split along K into fixed-order partial sums; no float atomics)
// mode 1 reproduces the CPU backend's literal arithmetic for the gradients (see include/ferrox_hip.h).
#include <cstdlib>

#include "igemm_core.hpp"
#include "gemm_lds.hpp"
#include "wgrad_patch.hpp"
#include "wgrad_patch_s2.hpp"
#include "dgrad_patch_s2.hpp"
#include "dgrad_patch_s2_f64.hpp"
#include "fwd_patch_s2.hpp"
#include "fwd_patch_s2_f64.hpp"
#include "conv_smallc.hpp"
#include "conv_image_f64.hpp"
#include "conv_patch.hpp"
#include "conv_patch_f64.hpp"
#include "wgrad_patch_f64.hpp"
#include "wgrad_patch_s2_f64.hpp"

namespace fx {
int col2im_f32(fx_ctx*, const float*, float*, i64, i64, i64, i64, i64, i64, i64, i64, i64, i64, int);
int col2im_f64(fx_ctx*, const double*, double*, i64, i64, i64, i64, i64, i64, i64, i64, i64, i64, int);
}
extern "C" int fx_gemm_f32(fx_ctx*, int, int, int64_t, int64_t, int64_t, const float*, const float*, float*);
extern "C" int fx_gemm_f64(fx_ctx*, int, int, int64_t, int64_t, int64_t, const double*, const double*, double*);

namespace {
using namespace igemm;

typedef Tile<128, 128, 16, 64, 64> TileM128;  // 4 waves as 2x2, 64x64 each
typedef Tile<64, 128, 16, 64, 32> TileM64;    // 4 waves as 1x4, 64x32 each
typedef Tile<32, 256, 16, 32, 64> TileM32;    // 4 waves as 1x4, 32x64 each
typedef Tile<64, 64, 16, 32, 32> TileSmall;   // 4 waves as 2x2, 32x32 each
typedef Tile<32, 32, 16, 32, 32> TileTiny;    // one wave: first-layer weight gradients (Cout <= 32, Cin*kh*kw <= 32)
// FX_CONV_GENERIC=1 in the environment sends every shape to the implicit-GEMM kernels (A/B timing, debugging).
// What the last convolution call on this context ran (fx_conv2d_last_path): a fixed string per dispatch branch.
#define FX_TAKES(c, name) ((c)->last_conv_path = (name))
static bool generic_only() { const char* v = getenv("FX_CONV_GENERIC"); return v && atoi(v) != 0; }

int gemm_t(fx_ctx* c, int ta, int tb, i64 M, i64 N, i64 K, const float* A, const float* B, float* C) { return fx_gemm_f32(c, ta, tb, M, N, K, A, B, C); }
int gemm_t(fx_ctx* c, int ta, int tb, i64 M, i64 N, i64 K, const double* A, const double* B, double* C) { return fx_gemm_f64(c, ta, tb, M, N, K, A, B, C); }
int col2im_t(fx_ctx* c, const float* col, float* out, i64 B, i64 C, i64 H, i64 W, i64 kh, i64 kw, i64 sh, i64 sw, i64 ph, i64 pw, int layout) { return fx::col2im_f32(c, col, out, B, C, H, W, kh, kw, sh, sw, ph, pw, layout); }
int col2im_t(fx_ctx* c, const double* col, double* out, i64 B, i64 C, i64 H, i64 W, i64 kh, i64 kw, i64 sh, i64 sw, i64 ph, i64 pw, int layout) { return fx::col2im_f64(c, col, out, B, C, H, W, kh, kw, sh, sw, ph, pw, layout); }

inline bool aligned16(const void* a, const void* b) { return (((uintptr_t)a | (uintptr_t)b) & 15) == 0; }

struct Dims {
    i64 B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, oh, ow;
    i64 bc;  // images per launch: the kernels index one launch's tensors with 32-bit byte offsets and pixel numbers
};

template <typename T>
int check_dims(Dims& d, i64 B, i64 Cin, i64 H, i64 W, i64 Cout, i64 kh, i64 kw, i64 sh, i64 sw, i64 ph, i64 pw, const char* what) {
    FX_REQUIRE(B > 0 && Cin > 0 && H > 0 && W > 0 && Cout > 0 && kh > 0 && kw > 0 && sh > 0 && sw > 0 && ph >= 0 && pw >= 0,
               "%s: non-positive dimension", what);
    FX_REQUIRE(H + 2 * ph >= kh && W + 2 * pw >= kw, "%s: kernel larger than padded input", what);
    FX_REQUIRE(ph < 32768 && pw < 32768 && kh < 32768 && kw < 32768, "%s: kernel/padding too large", what);
    d = Dims{B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, (H + 2 * ph - kh) / sh + 1, (W + 2 * pw - kw) / sw + 1, 0};
    const i64 lim = (1ll << 31) - 1;
    FX_REQUIRE(Cin * kh * kw <= lim && Cout * kh * kw <= lim, "%s: a GEMM dimension exceeds 2^31-1", what);
    // A batch whose tensors reach 2 GiB runs as several launches over slices of the batch (images are independent in
    // the forward pass and the data gradient; the weight gradient adds the slices' results in order).
    const i64 per_image = std::max(Cin * H * W, Cout * d.oh * d.ow) * (i64)sizeof(T);
    if (per_image > lim) {
        fx::set_error("%s: one image of 2 GiB or more is not supported by this build", what);
        return FX_ERR_UNSUPPORTED;
    }
    d.bc = std::min(B, lim / per_image);
    return FX_OK;
}

// Weight re-layouts feeding the A operand (w is [Cout][Cin][KK], KK = kh*kw):
//  mode 0: out[oc][r*Cin + c]   = w[oc][c][r]   forward, K ordered (ky,kx) outer / channel inner
//  mode 1: out[c][oc*KK + r]    = w[oc][c][r]   data gradient, K ordered like the reference (oc,ky,kx)
//  mode 2: out[c][r*Cout + oc]  = w[oc][c][r]   data gradient, K ordered (ky,kx) outer / out-channel inner
template <typename T>
__global__ __launch_bounds__(256) void permute_weights_kernel(const T* __restrict__ w, T* __restrict__ out, int Cout, int Cin, int KK, int mode) {
    const i64 i = (i64)blockIdx.x * 256 + threadIdx.x;
    const i64 n = (i64)Cout * Cin * KK;
    if (i >= n) return;
    int oc, c, r;
    if (mode == 0) { c = (int)(i % Cin); const i64 t = i / Cin; r = (int)(t % KK); oc = (int)(t / KK); }
    else if (mode == 1) { r = (int)(i % KK); const i64 t = i / KK; oc = (int)(t % Cout); c = (int)(t / Cout); }
    else { oc = (int)(i % Cout); const i64 t = i / Cout; r = (int)(t % KK); c = (int)(t / KK); }
    out[i] = w[((i64)oc * Cin + c) * KK + r];
}

template <typename T>
int permute_weights(fx_ctx* c, const T* w, T* out, const Dims& d, int mode) {
    const i64 nw = d.Cin * d.Cout * d.kh * d.kw;
    FX_LAUNCH(dim3((unsigned)fx::ceil_div(nw, 256)), dim3(256), 0, c->stream, (w, out, (int)d.Cout, (int)d.Cin, (int)(d.kh * d.kw), mode), permute_weights_kernel<T>);
    FX_LAUNCH_CHECK();
    return FX_OK;
}

// Tile for an [M x N] implicit GEMM without split-K: the widest tile that fits M, stepped down while the grid
// would leave CUs idle (a 14x14 layer at batch 32 has only 98 tiles of 128x128).  Returns 128, 64, 32 or 0 (64x64).
inline int pick_tile(fx_ctx* c, i64 M, i64 N) {
    const i64 cus = c ? c->num_cus : 256;
    if (M > 64) {
        if (fx::ceil_div(M, (i64)128) * fx::ceil_div(N, (i64)128) >= cus) return 128;
        if (fx::ceil_div(M, (i64)64) * fx::ceil_div(N, (i64)128) >= cus) return 64;
        return 0;
    }
    if (M > 32) return fx::ceil_div(N, (i64)128) >= cus ? 64 : 0;
    return 32;
}

constexpr int CONV_BK = 16;  // slab depth of every conv tile; the (ky,kx)-outer K order needs channels % CONV_BK == 0

template <typename T, class Cfg, bool FAST>
int fwd_tile(fx_ctx* c, const T* x, const T* w, T* y, const Dims& d, const T* bias, int relu) {
    static_assert(Cfg::BK == CONV_BK || !FAST || Cfg::BK == 32, "unexpected slab depth");
    const i64 M = d.Cout, N = d.B * d.oh * d.ow, K = d.Cin * d.kh * d.kw;
    const ConvShape s = make_shape(d.B, d.Cin, d.H, d.W, d.Cout, d.kh, d.kw, d.sh, d.sw, d.ph, d.pw);
    MatLoader<T, true> al{w, K, (int)M};
    ConvFwdB<T, FAST> bl{x, s, (int)N};
    const int kps = (int)(fx::ceil_div(K, Cfg::BK) * Cfg::BK);
    if (bias) {
        NchwStore<T, true> ep{y, (int)d.Cout, (int)(d.oh * d.ow), (int)N, s.div_L, bias, relu};
        return launch<T, Cfg>(c, al, bl, ep, M, N, K, 1, kps);
    }
    NchwStore<T> ep{y, (int)d.Cout, (int)(d.oh * d.ow), (int)N, s.div_L};
    return launch<T, Cfg>(c, al, bl, ep, M, N, K, 1, kps);
}

// Image layers (at most 4 input channels forward, 3 for the weight gradient), f32 3x3.
template <typename T>
csc::Plan smallc_plan(fx_ctx* c, const Dims& d, bool wgrad) {
    if constexpr (sizeof(T) == 4) {
        if (!generic_only()) return csc::make_plan(c ? c->num_cus : 256, wgrad, d.B, d.Cin, d.H, d.W, d.Cout, d.kh, d.kw, d.sh, d.sw, d.ph, d.pw, d.oh, d.ow);
    }
    return csc::Plan();
}

template <typename T>
cpk::Plan fwd_patch_plan(fx_ctx* c, const Dims& d) {
    if constexpr (sizeof(T) == 4) {
        if (!generic_only()) return cpk::make_plan(c ? c->num_cus : 256, d.B, d.Cin, d.H, d.W, d.Cout, d.oh, d.ow, d.kh, d.kw, d.sh, d.sw, d.ph, d.pw);
    }
    return cpk::Plan();
}

// The stride-1 data gradient is a forward pass over grad_out with padding k-1-p.
template <typename T>
cpk::Plan dgrad_patch_plan(fx_ctx* c, const Dims& d, int mode) {
    if constexpr (sizeof(T) == 4) {
        if (mode == 0 && !generic_only() && d.sh == 1 && d.sw == 1 && d.ph <= 2 && d.pw <= 2)
            return cpk::make_plan(c ? c->num_cus : 256, d.B, d.Cout, d.oh, d.ow, d.Cin, d.H, d.W, d.kh, d.kw, 1, 1, 2 - d.ph, 2 - d.pw);
    }
    return cpk::Plan();
}

// f64: the same structure on the 16x16x4 MFMA (conv_patch_f64.hpp)
template <typename T>
cpd::Plan fwd_patch64_plan(fx_ctx* c, const Dims& d) {
    if constexpr (sizeof(T) == 8) {
        if (!generic_only()) return cpd::make_plan(c ? c->num_cus : 256, d.B, d.Cin, d.H, d.W, d.Cout, d.oh, d.ow, d.kh, d.kw, d.sh, d.sw, d.ph, d.pw);
    }
    return cpd::Plan();
}
template <typename T>
cpd::Plan dgrad_patch64_plan(fx_ctx* c, const Dims& d, int mode) {
    if constexpr (sizeof(T) == 8) {
        if (mode == 0 && !generic_only() && d.sh == 1 && d.sw == 1 && d.ph <= 2 && d.pw <= 2)
            return cpd::make_plan(c ? c->num_cus : 256, d.B, d.Cout, d.oh, d.ow, d.Cin, d.H, d.W, d.kh, d.kw, 1, 1, 2 - d.ph, 2 - d.pw);
    }
    return cpd::Plan();
}

// 1x1 filters at unit stride without padding (f32): the convolution of one image is a plain product over the channels,
//   fwd    Y_b [Cout, L]  = W [Cout, Cin] . X_b [Cin, L]
//   dgrad  dX_b [Cin, L]  = W^T . G_b [Cout, L]
//   wgrad  dW [Cout, Cin] = sum over b of G_b [Cout, L] . X_b^T
// with every operand already laid out as the LDS-slab GEMM wants it (gemm_lds.hpp), so the whole batch runs as one launch of
// that kernel (blockIdx.y = image); the weight gradient leaves one partial product per image and the ordered sum adds them.
// kind: FX_CONV_FWD / FX_CONV_DGRAD / FX_CONV_WGRAD.
template <typename T>
glk::Plan pointwise_plan(fx_ctx* c, const Dims& d, int kind) {
    if constexpr (sizeof(T) == 4) {
        if (generic_only() || d.kh != 1 || d.kw != 1 || d.sh != 1 || d.sw != 1 || d.ph != 0 || d.pw != 0 || d.B > 65535) return glk::Plan();
        const int cus = c ? c->num_cus : 256;
        const i64 L = d.H * d.W;
        glk::Plan pl;
        if (kind == FX_CONV_FWD) pl = glk::make_plan(cus, false, false, d.Cout, L, d.Cin, d.Cin, L, d.B);
        else if (kind == FX_CONV_DGRAD) pl = glk::make_plan(cus, true, false, d.Cin, L, d.Cout, d.Cin, L, d.B);
        // (one partial result per image: where those outweigh the operands -- small maps under many channels -- the implicit GEMM's
        // K split over the whole batch moves less; measured at [64,1024,14,14] -> 256: 63 against 66 TFLOP/s, at [64,256,14,14] -> 256: 46 against 31)
        else if (d.B * d.Cout * d.Cin <= 0x7fffffff && 5 * d.Cout * d.Cin <= 4 * (d.Cout + d.Cin) * L)
            pl = glk::make_plan(cus, false, true, d.Cout, d.Cin, L, L, L, d.B);
        // only with the 128-row tiles: the 64-row ones measured below the implicit GEMM here ([32,256,56,56] -> 64: 55 against
        // 63 TFLOP/s forward), the 128-row ones above it (-> 256: 92 against 86; [16,256,16,16] -> 1024: 94 against 64)
        return pl.ok && pl.WM == 4 ? pl : glk::Plan();
    }
    return glk::Plan();
}

template <typename T>
i64 fwd_ws_bytes(fx_ctx* c, const Dims& d) {
    // enough for either kernel: a misaligned tensor sends a patch-kernel shape to the implicit GEMM
    const cpk::Plan pl = fwd_patch_plan<T>(c, d);
    const i64 generic = d.Cin % CONV_BK == 0 ? d.Cin * d.Cout * d.kh * d.kw * (i64)sizeof(T) : 0;
    const cpd::Plan pd = fwd_patch64_plan<T>(c, d);
    if (pd.ok) return std::max(generic, cpd::workspace_bytes(pd));
    return pl.ok ? std::max(generic, cpk::workspace_bytes(pl, d.Cout)) : generic;
}

template <typename T>
int conv_fwd(fx_ctx* c, const T* x, const T* w, T* y, i64 B, i64 Cin, i64 H, i64 W, i64 Cout, i64 kh, i64 kw, i64 sh, i64 sw,
             i64 ph, i64 pw, void* ws, i64 ws_bytes, const T* bias = nullptr, int relu = 0) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(x && w && y, "fx_conv2d_fwd: null pointer");
    Dims d;
    if (int rc = check_dims<T>(d, B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, "fx_conv2d_fwd")) return rc;
    if (d.B > d.bc) {  // slices of the batch, one launch sequence each
        for (i64 b0 = 0; b0 < B; b0 += d.bc) {
            const i64 nb = std::min(d.bc, B - b0);
            if (int rc = conv_fwd<T>(c, x + b0 * Cin * H * W, w, y + b0 * Cout * d.oh * d.ow, nb, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw,
                                     ws, ws_bytes, bias, relu))
                return rc;
        }
        return FX_OK;
    }
    const i64 need = fwd_ws_bytes<T>(c, d);
    FX_REQUIRE(ws == nullptr || ws_bytes >= need, "fx_conv2d_fwd: workspace of %lld bytes is smaller than the %lld needed",
               (long long)ws_bytes, (long long)need);
    std::lock_guard<std::mutex> lk(c->launch_mutex);
    if constexpr (sizeof(T) == 4) {
        const csc::Plan sp = smallc_plan<T>(c, d, false);
        if (sp.ok && aligned16(x, x)) return FX_TAKES(c, "image layer, tiles (csc)"), csc::run_fwd(c, sp, x, w, y, B, Cin, H, W, Cout, d.oh, d.ow, sh, sw, ph, pw, bias, relu);
        if (!generic_only()) {
            const fw2::Plan f2 = fw2::make_plan(d.B, d.Cin, d.H, d.W, d.Cout, d.kh, d.kw, d.sh, d.sw, d.ph, d.pw, d.oh, d.ow);
            if (f2.ok && aligned16(x, w) && aligned16(y, y)) return FX_TAKES(c, "stride-2 patch (fw2)"), fw2::run(c, f2, x, w, y, B, Cin, H, Cout, d.oh, bias, relu);
        }
        const glk::Plan pp = pointwise_plan<T>(c, d, FX_CONV_FWD);
        if (pp.ok && aligned16(x, w) && aligned16(y, y)) {
            const i64 L = d.H * d.W;
            return FX_TAKES(c, "1x1 as batched slab GEMM (glk)"), glk::run(c, pp, false, false, Cout, L, Cin, w, x, y, bias, relu, B, 0, Cin * L, Cout * L, 1);
        }
        const cpk::Plan pl = fwd_patch_plan<T>(c, d);
        if (pl.ok && aligned16(x, ws)) {
            float* wimg = (float*)(ws ? ws : c->get_scratch(need));
            if (!wimg) return FX_ERR_OOM;
            return FX_TAKES(c, "LDS patch (cpk)"), cpk::run(c, pl, x, w, y, wimg, 0, Cout, Cin, B, Cin, H, W, Cout, d.oh, d.ow, sh, sw, ph, pw, bias, relu);
        }
    }
    if constexpr (sizeof(T) == 8) {
        if (!generic_only() && cim::eligible(d.B, d.Cin, d.H, d.W, d.Cout, d.kh, d.kw, d.sh, d.sw, d.ph, d.pw) && aligned16(x, x) && aligned16(y, y))
            return FX_TAKES(c, "image layer (cim)"), cim::run(c, x, w, y, B, Cin, H, Cout, bias, relu);
        if (!generic_only()) {
            const fwd2::Plan f2 = fwd2::make_plan(d.B, d.Cin, d.H, d.W, d.Cout, d.kh, d.kw, d.sh, d.sw, d.ph, d.pw, d.oh, d.ow);
            if (f2.ok && aligned16(x, w) && aligned16(y, y)) return FX_TAKES(c, "stride-2 patch (fwd2)"), fwd2::run(c, f2, x, w, y, B, Cin, H, Cout, d.oh, bias, relu);
        }
        const cpd::Plan pd = fwd_patch64_plan<T>(c, d);
        if (pd.ok && aligned16(x, ws) && aligned16(y, y)) {
            double* wimg = (double*)(ws ? ws : c->get_scratch(need));
            if (!wimg) return FX_ERR_OOM;
            return FX_TAKES(c, "LDS patch (cpd)"), cpd::run(c, pd, x, w, y, wimg, 0, Cout, Cin, B, Cin, H, W, Cout, d.oh, d.ow, sh, sw, ph, pw, bias, relu);
        }
    }
    FX_TAKES(c, "implicit GEMM");
    if (d.Cin % CONV_BK == 0) {
        T* wp = (T*)(ws ? ws : c->get_scratch(need));
        if (!wp) return FX_ERR_OOM;
        if (int rc = permute_weights<T>(c, w, wp, d, 0)) return rc;
        switch (pick_tile(c, Cout, B * d.oh * d.ow)) {
            case 128: return fwd_tile<T, TileM128, true>(c, x, wp, y, d, bias, relu);
            case 64: return fwd_tile<T, TileM64, true>(c, x, wp, y, d, bias, relu);
            case 32: return fwd_tile<T, TileM32, true>(c, x, wp, y, d, bias, relu);
            default: return fwd_tile<T, TileSmall, true>(c, x, wp, y, d, bias, relu);
        }
    }
    switch (pick_tile(c, Cout, B * d.oh * d.ow)) {
        case 128: return fwd_tile<T, TileM128, false>(c, x, w, y, d, bias, relu);
        case 64: return fwd_tile<T, TileM64, false>(c, x, w, y, d, bias, relu);
        case 32: return fwd_tile<T, TileM32, false>(c, x, w, y, d, bias, relu);
        default: return fwd_tile<T, TileSmall, false>(c, x, w, y, d, bias, relu);
    }
}

template <typename T, class Cfg, bool FAST>
int dgrad_tile(fx_ctx* c, const T* g, const T* wt, T* dx, const Dims& d) {
    const i64 M = d.Cin, N = d.B * d.H * d.W, K = d.Cout * d.kh * d.kw;
    const ConvShape s = make_shape(d.B, d.Cin, d.H, d.W, d.Cout, d.kh, d.kw, d.sh, d.sw, d.ph, d.pw);
    MatLoader<T, true> al{wt, K, (int)M};
    ConvDgradB<T, FAST> bl{g, s, (int)N};
    NchwStore<T> ep{dx, (int)d.Cin, (int)(d.H * d.W), (int)N, s.div_HW};
    const int kps = (int)(fx::ceil_div(K, Cfg::BK) * Cfg::BK);
    return launch<T, Cfg>(c, al, bl, ep, M, N, K, 1, kps);
}

// Strided data gradient by pixel classes.  An input pixel (y, x) only receives taps with ky = (y+ph) mod sh and
// kx = (x+pw) mod sw (mod the strides), so the gather over all kh*kw taps multiplies mostly zeros (3 of 4 for a
// 3x3 stride-2 layer).  Pixels are grouped by (ry, rx) = ((y+ph) % sh, (x+pw) % sw); each class is a dense
// stride-1 correlation of grad_out with the sub-filter w[.., ry + jy*sh, rx + jx*sw] (flipped), written to the
// class's sub-grid of dx.  One implicit GEMM per class, with exactly the useful multiply-adds.
//   out[c][yy][xx] = sum_{j'y, j'x, oc} g[oc][yy - pad_y + j'y][xx - pad_x + j'x] * wcls[c][(j'y, j'x, oc)]
constexpr int MAX_CLASSES = 4;  // sh * sw pixel classes handled in one launch (stride 2 in both directions)
struct ClassPerm {
    int ry[MAX_CLASSES], rx[MAX_CLASSES], nky[MAX_CLASSES], nkx[MAX_CLASSES];
    i64 offset[MAX_CLASSES], n[MAX_CLASSES];
};
// Sub-filters of all classes, one launch: blockIdx.y = class; out[offset + ((c*nky + jy)*nkx + jx)*Cout + oc].
template <typename T>
__global__ __launch_bounds__(256) void permute_weights_class_kernel(const T* __restrict__ w, T* __restrict__ out, int Cout, int Cin, int kh,
                                                                    int kw, int sh, int sw, const ClassPerm cp) {
    const int z = blockIdx.y;
    const i64 i = (i64)blockIdx.x * 256 + threadIdx.x;
    if (i >= cp.n[z]) return;
    const int nky = cp.nky[z], nkx = cp.nkx[z];
    const int oc = (int)(i % Cout);
    i64 t = i / Cout;
    const int jx = (int)(t % nkx);
    t /= nkx;
    const int jy = (int)(t % nky), c = (int)(t / nky);
    const int ky = cp.ry[z] + (nky - 1 - jy) * sh, kx = cp.rx[z] + (nkx - 1 - jx) * sw;
    out[cp.offset[z] + i] = w[(((i64)oc * Cin + c) * kh + ky) * kw + kx];
}

template <typename T>
bool dgrad_classes_ok(const Dims& d) {
    return (d.sh > 1 || d.sw > 1) && d.kh >= d.sh && d.kw >= d.sw && d.Cout % CONV_BK == 0 && !generic_only();
}

// One class = one forward stride-1 correlation over grad_out with the class's sub-filter, stored to the class's
// sub-grid of dx.  Classes go out MAX_CLASSES per launch (blockIdx.z = class): each alone is a small GEMM (a quarter
// of the pixels for stride 2) that fills only part of the chip.
template <typename T, class Cfg>
int dgrad_classes_tile(fx_ctx* c, const T* g, const T* w, T* dx, T* wt, const Dims& d) {
    typedef igemm::MultiProblem<MatLoader<T, true>, ConvFwdB<T, true>, NchwSubgridStore<T>, MAX_CLASSES> MP;
    MP mp;
    ClassPerm cp;
    int count = 0;
    i64 woff = 0, max_n = 0;
    auto flush = [&]() -> int {
        if (count == 0) return FX_OK;
        FX_LAUNCH(dim3((unsigned)fx::ceil_div(max_n, 256), (unsigned)count), dim3(256), 0, c->stream, (
            w, wt, (int)d.Cout, (int)d.Cin, (int)d.kh, (int)d.kw, (int)d.sh, (int)d.sw, cp), permute_weights_class_kernel<T>);
        FX_LAUNCH_CHECK();
        const int rc = igemm::launch_multi<T, Cfg>(c, mp, count);
        count = 0;
        max_n = 0;
        return rc;
    };
    for (int ry = 0; ry < d.sh; ++ry)
        for (int rx = 0; rx < d.sw; ++rx) {
            const int y0 = (int)(((ry - d.ph) % d.sh + d.sh) % d.sh), x0 = (int)(((rx - d.pw) % d.sw + d.sw) % d.sw);
            if (y0 >= d.H || x0 >= d.W) continue;  // no pixel of this class
            const int Hy = (int)((d.H - y0 + d.sh - 1) / d.sh), Wx = (int)((d.W - x0 + d.sw - 1) / d.sw);
            const int nky = (int)((d.kh - ry + d.sh - 1) / d.sh), nkx = (int)((d.kw - rx + d.sw - 1) / d.sw);
            const int dy0 = (int)((y0 + d.ph - ry) / d.sh), dx0 = (int)((x0 + d.pw - rx) / d.sw);
            const i64 nw = d.Cin * nky * nkx * d.Cout;
            // the class as a forward stride-1 correlation: input = grad_out [B, Cout, oh, ow], kernel nky x nkx
            ConvShape s = make_shape(d.B, d.Cout, d.oh, d.ow, d.Cin, nky, nkx, 1, 1, 0, 0);
            s.ph = (nky - 1) - dy0;
            s.pw = (nkx - 1) - dx0;
            s.oh = Hy;
            s.ow = Wx;
            s.div_L = FastDiv((uint32_t)(Hy * Wx));
            s.div_ow = FastDiv((uint32_t)Wx);
            const i64 M = d.Cin, N = d.B * Hy * Wx, K = (i64)nky * nkx * d.Cout;
            const int z = count++;
            cp.ry[z] = ry; cp.rx[z] = rx; cp.nky[z] = nky; cp.nkx[z] = nkx; cp.offset[z] = woff; cp.n[z] = nw;
            max_n = std::max(max_n, nw);
            mp.al[z] = MatLoader<T, true>{wt + woff, K, (int)M};
            mp.bl[z] = ConvFwdB<T, true>{g, s, (int)N};
            mp.ep[z] = NchwSubgridStore<T>{dx, (int)d.Cin, (int)d.H, (int)d.W, Hy, Wx, y0, x0, (int)d.sh, (int)d.sw, (int)N,
                                          FastDiv((uint32_t)(Hy * Wx)), FastDiv((uint32_t)Wx)};
            mp.K[z] = (int)K;
            mp.kps[z] = (int)(fx::ceil_div(K, Cfg::BK) * Cfg::BK);
            mp.tiles_n[z] = (int)fx::ceil_div(N, Cfg::BN);
            mp.tiles_m[z] = (int)fx::ceil_div(M, Cfg::BM);
            woff += nw;
            if (count == MAX_CLASSES)
                if (int rc = flush()) return rc;
        }
    return flush();
}

template <typename T>
int dgrad_classes(fx_ctx* c, const T* g, const T* w, T* dx, T* wt, const Dims& d) {
    // tile from the largest class; all classes of one call share it
    const i64 Hy = fx::ceil_div(d.H, d.sh), Wx = fx::ceil_div(d.W, d.sw);
    switch (pick_tile(c, d.Cin, d.B * Hy * Wx * std::min<i64>(MAX_CLASSES, d.sh * d.sw))) {
        case 128: return dgrad_classes_tile<T, TileM128>(c, g, w, dx, wt, d);
        case 64: return dgrad_classes_tile<T, TileM64>(c, g, w, dx, wt, d);
        case 32: return dgrad_classes_tile<T, TileM32>(c, g, w, dx, wt, d);
        default: return dgrad_classes_tile<T, TileSmall>(c, g, w, dx, wt, d);
    }
}

// Data gradient for at most 4 input channels (the first layer of an image network): the implicit GEMM would pad
// Cin = 3 to a 32-row tile and run at 10 % useful work.  One thread owns one input pixel and all its channels and
// gathers over (tap, oc); the filters sit in LDS as wl[tap][oc][4] so one 16-byte broadcast read feeds the channel
// FMAs, and lanes walk consecutive x, so every grad_out load is a contiguous 256-byte row segment.
template <typename T>
__global__ __launch_bounds__(256) void dgrad_small_cin_kernel(const T* __restrict__ g, const T* __restrict__ w, T* __restrict__ dx,
                                                              ConvShape s, int npix) {
    FX_DYNAMIC_SMEM(unsigned char, smem_raw);
    T* wl = reinterpret_cast<T*>(smem_raw);
    const int KK = s.kh * s.kw;
    for (int i = threadIdx.x; i < KK * s.Cout * 4; i += 256) {
        const int c = i & 3, oc = (i >> 2) % s.Cout, t = (i >> 2) / s.Cout;
        wl[i] = c < s.Cin ? w[((i64)oc * s.Cin + c) * KK + t] : T(0);
    }
    __syncthreads();
    const int n = blockIdx.x * 256 + threadIdx.x;
    if (n >= npix) return;
    const uint32_t b = s.div_HW.div((uint32_t)n), rem = n - b * (s.H * s.W);
    const uint32_t y = s.div_W.div(rem), x = rem - y * s.W;
    const int L = s.oh * s.ow;
    const T* gb = g + (i64)b * s.Cout * L;
    T acc[4] = {T(0), T(0), T(0), T(0)};
    for (int ky = 0; ky < s.kh; ++ky) {
        const int ty = (int)y + s.ph - ky;
        if (ty < 0) continue;
        const uint32_t oy = s.div_sh.div((uint32_t)ty);
        if ((int)(oy * s.sh) != ty || (int)oy >= s.oh) continue;
        for (int kx = 0; kx < s.kw; ++kx) {
            const int tx = (int)x + s.pw - kx;
            if (tx < 0) continue;
            const uint32_t ox = s.div_sw.div((uint32_t)tx);
            if ((int)(ox * s.sw) != tx || (int)ox >= s.ow) continue;
            const T* gp = gb + oy * s.ow + ox;
            const T* wt = wl + (ky * s.kw + kx) * s.Cout * 4;
#pragma unroll 4
            for (int oc = 0; oc < s.Cout; ++oc) {
                const T gv = gp[(i64)oc * L];
#pragma unroll
                for (int c = 0; c < 4; ++c) acc[c] += gv * wt[oc * 4 + c];
            }
        }
    }
    T* o = dx + (i64)b * s.Cin * s.H * s.W + rem;
    for (int c = 0; c < s.Cin; ++c) o[(i64)c * s.H * s.W] = acc[c];
}

// The same for 3 x 3 filters at unit stride and padding 1 over rows that are whole 16-byte vectors: a thread owns four consecutive
// input pixels of a row and reads the four grad_out values above them as one vector -- the two neighbours come from the adjacent
// lanes -- so one coalesced load feeds 3 x 4 x CIN FMAs (the kernel above: one load per CIN).  The output channels are split over
// the four waves of a block (wave q takes every fourth one), so four waves per SIMD hide the load latency; their sums are added
// through LDS in wave order.  A block covers 64 pixel groups.
// Measured on [256,3,32,32] <- 32 channels: 17.4 us against 31.1 us with the kernel above; with four pixels per thread read as six
// scalar loads (lanes 16 bytes apart: four times the cache lines per load) 38.0 us.
__device__ __forceinline__ void load4(const float* p, float (&v)[4]) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
__device__ __forceinline__ void load4(const double* p, double (&v)[4]) {
    const double2 t0 = *reinterpret_cast<const double2*>(p), t1 = *reinterpret_cast<const double2*>(p + 2);
    v[0] = t0.x; v[1] = t0.y; v[2] = t1.x; v[3] = t1.y;
}
template <typename T, int CIN>
__global__ __launch_bounds__(256) void dgrad_small_cin_s1_kernel(const T* __restrict__ g, const T* __restrict__ w, T* __restrict__ dx,
                                                                 ConvShape s, int ngroups, int WQ, igemm::FastDiv div_wq) {
    constexpr int KW = 3, PX = 4;
    FX_DYNAMIC_SMEM(unsigned char, smem_raw);
    T* wl = reinterpret_cast<T*>(smem_raw);  // [tap][oc][4]; afterwards the sums of waves 1 .. 3: [3][PX * CIN][64]
    const int KK = 3 * KW;
    for (int i = threadIdx.x; i < KK * s.Cout * 4; i += 256) {
        const int c = i & 3, oc = (i >> 2) % s.Cout, t = (i >> 2) / s.Cout;
        wl[i] = c < s.Cin ? w[((i64)oc * s.Cin + c) * KK + t] : T(0);
    }
    __syncthreads();
    const int lane = threadIdx.x & 63, q = threadIdx.x >> 6;
    const int n = blockIdx.x * 64 + lane;
    const bool live = n < ngroups;
    const uint32_t nn = live ? (uint32_t)n : 0u;
    const uint32_t row = div_wq.div(nn), xq = nn - row * WQ;  // row = b * H + y
    const uint32_t b = row / (uint32_t)s.H;
    const int y = (int)(row - b * s.H), x0 = (int)xq * PX;
    const int L = s.H * s.W;  // the output map has the size of the input
    const T* gb = g + (i64)b * s.Cout * L + x0;
    // the values left and right of the vector: from the neighbouring lane when it holds the same row, else (a row that continues
    // in another wave) loaded by this lane; zero outside the row
    const bool has_left = xq > 0, has_right = (int)xq < WQ - 1;
    const bool left_far = live && has_left && lane == 0, right_far = live && has_right && (lane == 63 || n + 1 >= ngroups);
    T acc[PX][CIN];
#pragma unroll
    for (int j = 0; j < PX; ++j)
#pragma unroll
        for (int c = 0; c < CIN; ++c) acc[j][c] = T(0);
    for (int ky = 0; ky < 3; ++ky) {
        const int oy = y + 1 - ky;
        if (oy < 0 || oy >= s.H) continue;
        const T* grow = gb + (i64)oy * s.W;
        const T* wrow = wl + ky * KW * s.Cout * 4;
#pragma unroll 2
        for (int oc = q; oc < s.Cout; oc += 4) {
            T gv[KW + PX - 1], mid[4];
            const T* gp = grow + (i64)oc * L;
            if (live) load4(gp, mid);
            else mid[0] = mid[1] = mid[2] = mid[3] = T(0);
            T lv = __shfl_up(mid[3], 1, 64), rv = __shfl_down(mid[0], 1, 64);
            if (left_far) lv = gp[-1];
            if (right_far) rv = gp[4];
            gv[0] = has_left ? lv : T(0);
            gv[1] = mid[0]; gv[2] = mid[1]; gv[3] = mid[2]; gv[4] = mid[3];
            gv[5] = has_right ? rv : T(0);
#pragma unroll
            for (int kx = 0; kx < KW; ++kx) {
                const T* wt = wrow + (kx * s.Cout + oc) * 4;
#pragma unroll
                for (int c = 0; c < CIN; ++c) {
                    const T wv = wt[c];
#pragma unroll
                    for (int j = 0; j < PX; ++j) acc[j][c] += gv[j + KW - 1 - kx] * wv;  // grad_out column x0 + j + 1 - kx
                }
            }
        }
    }
    __syncthreads();  // every wave is done with the filters
    T* red = wl;
    if (q != 0) {
#pragma unroll
        for (int j = 0; j < PX; ++j)
#pragma unroll
            for (int c = 0; c < CIN; ++c) red[((q - 1) * PX * CIN + j * CIN + c) * 64 + lane] = acc[j][c];
    }
    __syncthreads();
    if (q != 0 || !live) return;
    T* o = dx + ((i64)b * s.Cin * s.H + y) * s.W + x0;
#pragma unroll
    for (int c = 0; c < CIN; ++c)
#pragma unroll
        for (int j = 0; j < PX; ++j) {
            T v = acc[j][c];
#pragma unroll
            for (int r = 0; r < 3; ++r) v += red[(r * PX * CIN + j * CIN + c) * 64 + lane];
            o[(i64)c * s.H * s.W + j] = v;
        }
}

template <typename T>
bool dgrad_small_cin_ok(const Dims& d) {
    return d.Cin <= 4 && d.kh * d.kw * d.Cout * 4 * (i64)sizeof(T) <= 48 * 1024 && !generic_only();
}

template <typename T>
int dgrad_small_cin(fx_ctx* c, const T* g, const T* w, T* dx, const Dims& d) {
    const ConvShape s = make_shape(d.B, d.Cin, d.H, d.W, d.Cout, d.kh, d.kw, d.sh, d.sw, d.ph, d.pw);
    const i64 npix = d.B * d.H * d.W;
    const size_t smem = (size_t)(d.kh * d.kw * d.Cout * 4) * sizeof(T);
    // (f64: level with the one-pixel kernel, 30.8 against 34.6 us on that layer and 242 against 210 us on [16,4,224,224] <- 64)
    if (sizeof(T) == 4 && d.sh == 1 && d.sw == 1 && d.kh == 3 && d.kw == 3 && d.ph == 1 && d.pw == 1 && d.W % 4 == 0 && d.Cin >= 3 &&
        fx::aligned16(g) && d.B * d.H * d.W < (1ll << 31)) {
        const i64 WQ = fx::ceil_div(d.W, (i64)4), ngroups = d.B * d.H * WQ;
        const size_t need = std::max(smem, (size_t)3 * 4 * d.Cin * 64 * sizeof(T));
        const dim3 grid((unsigned)fx::ceil_div(ngroups, (i64)64));
        const igemm::FastDiv div_wq((uint32_t)WQ);
        if (d.Cin == 3) FX_LAUNCH(grid, dim3(256), need, c->stream, (g, w, dx, s, (int)ngroups, (int)WQ, div_wq), dgrad_small_cin_s1_kernel<T, 3>);
        else FX_LAUNCH(grid, dim3(256), need, c->stream, (g, w, dx, s, (int)ngroups, (int)WQ, div_wq), dgrad_small_cin_s1_kernel<T, 4>);
        FX_LAUNCH_CHECK();
        return FX_OK;
    }
    FX_LAUNCH(dim3((unsigned)fx::ceil_div(npix, 256)), dim3(256), smem, c->stream, (g, w, dx, s, (int)npix), dgrad_small_cin_kernel<T>);
    FX_LAUNCH_CHECK();
    return FX_OK;
}

template <typename T>
i64 dgrad_ws_bytes(fx_ctx* c, const Dims& d, int mode) {
    if (mode == 1) return d.Cin * d.kh * d.kw * d.B * d.oh * d.ow * (i64)sizeof(T);
    const cpk::Plan pl = dgrad_patch_plan<T>(c, d, mode);
    const i64 generic = d.Cin * d.Cout * d.kh * d.kw * (i64)sizeof(T);
    const cpd::Plan pd = dgrad_patch64_plan<T>(c, d, mode);
    if (pd.ok) return std::max(generic, cpd::workspace_bytes(pd));
    return pl.ok ? std::max(generic, cpk::workspace_bytes(pl, d.Cin)) : generic;
}

template <typename T>
int conv_dgrad(fx_ctx* c, const T* g, const T* w, T* dx, i64 B, i64 Cin, i64 H, i64 W, i64 Cout, i64 kh, i64 kw, i64 sh, i64 sw,
               i64 ph, i64 pw, int mode, void* ws, i64 ws_bytes) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(g && w && dx, "fx_conv2d_dgrad: null pointer");
    FX_REQUIRE(mode == 0 || mode == 1, "fx_conv2d_dgrad: mode must be 0 or 1");
    Dims d;
    if (int rc = check_dims<T>(d, B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, "fx_conv2d_dgrad")) return rc;
    if (d.B > d.bc) {
        if (mode != 0) {  // the CPU-literal arithmetic reads grad_out flat across the whole batch
            fx::set_error("fx_conv2d_dgrad: mode 1 does not support tensors of 2 GiB or more");
            return FX_ERR_UNSUPPORTED;
        }
        for (i64 b0 = 0; b0 < B; b0 += d.bc) {
            const i64 nb = std::min(d.bc, B - b0);
            if (int rc = conv_dgrad<T>(c, g + b0 * Cout * d.oh * d.ow, w, dx + b0 * Cin * H * W, nb, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw,
                                       mode, ws, ws_bytes))
                return rc;
        }
        return FX_OK;
    }
    const i64 need = dgrad_ws_bytes<T>(c, d, mode);
    FX_REQUIRE(ws == nullptr || ws_bytes >= need, "fx_conv2d_dgrad: workspace of %lld bytes is smaller than the %lld needed",
               (long long)ws_bytes, (long long)need);
    if (mode == 1) {
        // CPU-literal arithmetic: col[K, N] = W2d^T . (g read flat as [Cout, N]); col2im with the batch-major index.
        const i64 K = Cin * kh * kw, N = B * d.oh * d.ow;
        T* col = (T*)ws;
        bool own = false;
        if (!col) {
            FX_NOT_RECORDING(c, "a convolution call without a caller-supplied workspace");
            FX_HIP_CHECK(hipMalloc((void**)&col, (size_t)need));
            own = true;
        }
        FX_TAKES(c, "explicit GEMM + col2im (CPU-literal mode)");
        int rc = gemm_t(c, 1, 0, K, N, Cout, w, g, col);
        if (!rc) rc = col2im_t(c, col, dx, B, Cin, H, W, kh, kw, sh, sw, ph, pw, 1);
        if (own) {
            (void)hipStreamSynchronize(c->stream);
            (void)hipFree(col);
        }
        return rc;
    }
    if (dgrad_small_cin_ok<T>(d)) return FX_TAKES(c, "direct gather, few input channels"), dgrad_small_cin<T>(c, g, w, dx, d);
    std::lock_guard<std::mutex> lk(c->launch_mutex);
    if constexpr (sizeof(T) == 4) {
        if (!generic_only()) {
            const dg2::Plan p2 = dg2::make_plan(d.B, d.Cin, d.H, d.W, d.Cout, d.kh, d.kw, d.sh, d.sw, d.ph, d.pw, d.oh, d.ow);
            if (p2.ok && aligned16(g, w) && aligned16(dx, dx)) return FX_TAKES(c, "stride-2 patch (dg2)"), dg2::run(c, p2, g, w, dx, B, Cin, Cout, d.oh);
            const glk::Plan pp = pointwise_plan<T>(c, d, FX_CONV_DGRAD);
            if (pp.ok && aligned16(g, w) && aligned16(dx, dx)) {
                const i64 L = d.H * d.W;
                return FX_TAKES(c, "1x1 as batched slab GEMM (glk)"), glk::run(c, pp, true, false, Cin, L, Cout, w, g, dx, nullptr, 0, B, 0, Cout * L, Cin * L);
            }
        }
    } else {
        if (!generic_only()) {
            const dgd2::Plan p2 = dgd2::make_plan(d.B, d.Cin, d.H, d.W, d.Cout, d.kh, d.kw, d.sh, d.sw, d.ph, d.pw, d.oh, d.ow);
            if (p2.ok && aligned16(g, w) && aligned16(dx, dx)) return FX_TAKES(c, "stride-2 patch (dgd2)"), dgd2::run(c, p2, g, w, dx, B, Cin, Cout, d.oh);
        }
    }
    T* wt = (T*)(ws ? ws : c->get_scratch(need));
    if (!wt) return FX_ERR_OOM;
    if constexpr (sizeof(T) == 4) {
        const cpk::Plan pl = dgrad_patch_plan<T>(c, d, mode);
        if (pl.ok && aligned16(g, wt)) return FX_TAKES(c, "LDS patch (cpk)"), cpk::run(c, pl, g, w, dx, wt, 1, Cout, Cin, B, Cout, d.oh, d.ow, Cin, H, W, 1, 1, 2 - ph, 2 - pw);
    }
    if constexpr (sizeof(T) == 8) {
        const cpd::Plan pd = dgrad_patch64_plan<T>(c, d, mode);
        if (pd.ok && aligned16(g, wt) && aligned16(dx, dx)) return FX_TAKES(c, "LDS patch (cpd)"), cpd::run(c, pd, g, w, dx, wt, 1, Cout, Cin, B, Cout, d.oh, d.ow, Cin, H, W, 1, 1, 2 - ph, 2 - pw);
    }
    if (dgrad_classes_ok<T>(d)) return FX_TAKES(c, "implicit GEMM by pixel classes"), dgrad_classes<T>(c, g, w, dx, wt, d);
    FX_TAKES(c, "implicit GEMM");
    if (Cout % CONV_BK == 0) {
        if (int rc = permute_weights<T>(c, w, wt, d, 2)) return rc;
        switch (pick_tile(c, Cin, B * H * W)) {
            case 128: return dgrad_tile<T, TileM128, true>(c, g, wt, dx, d);
            case 64: return dgrad_tile<T, TileM64, true>(c, g, wt, dx, d);
            case 32: return dgrad_tile<T, TileM32, true>(c, g, wt, dx, d);
            default: return dgrad_tile<T, TileSmall, true>(c, g, wt, dx, d);
        }
    }
    if (int rc = permute_weights<T>(c, w, wt, d, 1)) return rc;
    switch (pick_tile(c, Cin, B * H * W)) {
        case 128: return dgrad_tile<T, TileM128, false>(c, g, wt, dx, d);
        case 64: return dgrad_tile<T, TileM64, false>(c, g, wt, dx, d);
        case 32: return dgrad_tile<T, TileM32, false>(c, g, wt, dx, d);
        default: return dgrad_tile<T, TileSmall, false>(c, g, wt, dx, d);
    }
}

template <typename T, class Cfg>
void wgrad_plan(fx_ctx* c, const Dims& d, int* splits, int* kps) {
    const i64 M = d.Cout, N = d.Cin * d.kh * d.kw, K = d.B * d.oh * d.ow;
    const i64 tiles = fx::ceil_div(M, Cfg::BM) * fx::ceil_div(N, Cfg::BN);
    *splits = choose_splits(tiles, K, Cfg::BK, (i64)(c ? c->num_cus : 256) * 4, kps);
}

template <typename T, class Cfg>
int wgrad_tile(fx_ctx* c, const T* x, const T* g, T* dw, const Dims& d, int mode, void* ws) {
    const i64 M = d.Cout, N = d.Cin * d.kh * d.kw, K = d.B * d.oh * d.ow;
    const ConvShape s = make_shape(d.B, d.Cin, d.H, d.W, d.Cout, d.kh, d.kw, d.sh, d.sw, d.ph, d.pw);
    int splits, kps;
    wgrad_plan<T, Cfg>(c, d, &splits, &kps);
    T* part = dw;
    if (splits > 1) {
        part = (T*)(ws ? ws : c->get_scratch((i64)splits * M * N * (i64)sizeof(T)));
        if (!part) return FX_ERR_OOM;
    }
    ConvWgradB<T> bl{x, s, (int)N};
    MatStore<T> ep{part, N, M * N, (int)M, (int)N};
    int rc;
    if (mode == 1) {
        MatLoader<T, true> al{g, K, (int)M};  // g read flat as [Cout, B*L] (convolutions.rs:323-326)
        rc = launch<T, Cfg>(c, al, bl, ep, M, N, K, splits, kps);
    } else {
        ConvWgradA<T> al{g, s};
        rc = launch<T, Cfg>(c, al, bl, ep, M, N, K, splits, kps);
    }
    if (rc || splits == 1) return rc;
    return launch_splitk_reduce<T>(c, part, dw, M * N, splits);
}

template <typename T>
wgp::Plan patch_plan(fx_ctx* c, const Dims& d, int mode) {
    if constexpr (sizeof(T) == 4) {
        if (mode == 0 && !generic_only())
            return wgp::make_plan(c ? c->num_cus : 256, d.B, d.Cin, d.H, d.W, d.Cout, d.kh, d.kw, d.sh, d.sw, d.ph, d.pw, d.oh, d.ow);
    }
    return wgp::Plan();
}

template <typename T>
wg2::Plan patch_s2_plan(fx_ctx* c, const Dims& d, int mode) {
    if constexpr (sizeof(T) == 4) {
        if (mode == 0 && !generic_only())
            return wg2::make_plan(c ? c->num_cus : 256, d.B, d.Cin, d.H, d.W, d.Cout, d.kh, d.kw, d.sh, d.sw, d.ph, d.pw, d.oh, d.ow);
    }
    return wg2::Plan();
}

template <typename T>
wgd::Plan patch64_plan(fx_ctx* c, const Dims& d, int mode) {
    if constexpr (sizeof(T) == 8) {
        if (mode == 0 && !generic_only())
            return wgd::make_plan(c ? c->num_cus : 256, d.B, d.Cin, d.H, d.W, d.Cout, d.kh, d.kw, d.sh, d.sw, d.ph, d.pw, d.oh, d.ow);
    }
    return wgd::Plan();
}

template <typename T>
wgd2::Plan patch64_s2_plan(fx_ctx* c, const Dims& d, int mode) {
    if constexpr (sizeof(T) == 8) {
        if (mode == 0 && !generic_only())
            return wgd2::make_plan(c ? c->num_cus : 256, d.B, d.Cin, d.H, d.W, d.Cout, d.kh, d.kw, d.sh, d.sw, d.ph, d.pw, d.oh, d.ow);
    }
    return wgd2::Plan();
}

template <typename T>
i64 wgrad_ws_bytes(fx_ctx* c, const Dims& d, int mode) {
    const wgp::Plan pl = patch_plan<T>(c, d, mode);
    int splits, kps;
    if (d.Cout > 64 && d.Cin * d.kh * d.kw > 64) wgrad_plan<T, TileM128>(c, d, &splits, &kps);
    else if (d.Cout <= 32 && d.Cin * d.kh * d.kw <= 32) wgrad_plan<T, TileTiny>(c, d, &splits, &kps);
    else wgrad_plan<T, TileSmall>(c, d, &splits, &kps);
    i64 generic = splits > 1 ? (i64)splits * d.Cout * d.Cin * d.kh * d.kw * (i64)sizeof(T) : 0;
    if (mode == 0) {
        const csc::Plan sp = smallc_plan<T>(c, d, true);
        if (sp.ok) generic = std::max(generic, csc::wgrad_workspace_bytes(sp, d.Cout, d.Cin, true));  // covers the masked variant too
    }
    const wgd::Plan pd = patch64_plan<T>(c, d, mode);
    if (pd.ok) generic = std::max(generic, wgd::workspace_bytes(pd, d.Cout, d.Cin));
    const wg2::Plan p2 = patch_s2_plan<T>(c, d, mode);
    if (p2.ok) generic = std::max(generic, wg2::workspace_bytes(p2, d.Cout, d.Cin, true));
    const wgd2::Plan q2 = patch64_s2_plan<T>(c, d, mode);
    if (q2.ok) generic = std::max(generic, wgd2::workspace_bytes(q2, d.Cout, d.Cin, true));
    if (mode == 0 && pointwise_plan<T>(c, d, FX_CONV_WGRAD).ok) generic = std::max(generic, d.B * d.Cout * d.Cin * (i64)sizeof(T));
    if constexpr (sizeof(T) == 8) {
        if (mode == 0 && !generic_only()) {
            const cim::WPlan ip = cim::wgrad_plan(c ? c->num_cus : 256, d.B, d.Cin, d.H, d.W, d.Cout, d.kh, d.kw, d.sh, d.sw, d.ph, d.pw);
            if (ip.ok) generic = std::max(generic, cim::wgrad_workspace_bytes(ip, d.Cout, d.Cin, true));
        }
    }
    return pl.ok ? std::max(generic, wgp::workspace_bytes(pl, d.Cout, d.Cin)) : generic;
}

template <typename T>
int conv_wgrad(fx_ctx* c, const T* x, const T* g, T* dw, i64 B, i64 Cin, i64 H, i64 W, i64 Cout, i64 kh, i64 kw, i64 sh, i64 sw,
               i64 ph, i64 pw, int mode, void* ws, i64 ws_bytes) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(x && g && dw, "fx_conv2d_wgrad: null pointer");
    FX_REQUIRE(mode == 0 || mode == 1, "fx_conv2d_wgrad: mode must be 0 or 1");
    Dims d;
    if (int rc = check_dims<T>(d, B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, "fx_conv2d_wgrad")) return rc;
    if (d.B > d.bc) {
        if (mode != 0) {
            fx::set_error("fx_conv2d_wgrad: mode 1 does not support tensors of 2 GiB or more");
            return FX_ERR_UNSUPPORTED;
        }
        // one weight gradient per slice of the batch, then their sum in slice order (a rare, large case: the buffer for
        // the slices' results is allocated and released here)
        const i64 nchunks = fx::ceil_div(B, d.bc), nw = Cout * Cin * kh * kw;
        T* tmp = nullptr;
        FX_NOT_RECORDING(c, "a convolution call without a caller-supplied workspace");
        FX_HIP_CHECK(hipMalloc((void**)&tmp, (size_t)(nchunks * nw) * sizeof(T)));
        int rc = FX_OK;
        for (i64 i = 0; i < nchunks && !rc; ++i) {
            const i64 b0 = i * d.bc, nb = std::min(d.bc, B - b0);
            rc = conv_wgrad<T>(c, x + b0 * Cin * H * W, g + b0 * Cout * d.oh * d.ow, tmp + i * nw, nb, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw,
                               mode, ws, ws_bytes);
        }
        if (!rc) {
            std::lock_guard<std::mutex> lk(c->launch_mutex);
            rc = launch_splitk_reduce<T>(c, tmp, dw, nw, (int)nchunks);
        }
        (void)hipStreamSynchronize(c->stream);
        (void)hipFree(tmp);
        return rc;
    }
    const i64 need = wgrad_ws_bytes<T>(c, d, mode);
    FX_REQUIRE(ws == nullptr || ws_bytes >= need, "fx_conv2d_wgrad: workspace of %lld bytes is smaller than the %lld needed",
               (long long)ws_bytes, (long long)need);
    std::lock_guard<std::mutex> lk(c->launch_mutex);
    if constexpr (sizeof(T) == 4) {
        const csc::Plan sp = mode == 0 ? smallc_plan<T>(c, d, true) : csc::Plan();
        if (sp.ok && aligned16(x, g)) {
            float* part = nullptr;
            if (sp.splits > 1) {
                part = (float*)(ws ? ws : c->get_scratch(need));
                if (!part) return FX_ERR_OOM;
            }
            FX_TAKES(c, sp.rb ? "image layer, row bands (csc)" : "image layer, tiles (csc)");
            return csc::run_wgrad(c, sp, x, g, dw, part, Cin, H, W, Cout, d.oh, d.ow, sh, sw, ph, pw);
        }
        const wg2::Plan p2 = patch_s2_plan<T>(c, d, mode);
        if (p2.ok && aligned16(x, g) && aligned16(ws, ws)) {
            float* part = (float*)(ws ? ws : c->get_scratch(need));
            if (!part) return FX_ERR_OOM;
            return FX_TAKES(c, "stride-2 patch (wg2)"), wg2::run(c, p2, x, g, dw, part, Cin, H, Cout, ph, d.oh);
        }
        const glk::Plan pp = mode == 0 ? pointwise_plan<T>(c, d, FX_CONV_WGRAD) : glk::Plan();
        if (pp.ok && aligned16(x, g) && aligned16(ws, dw)) {
            const i64 L = d.H * d.W, n = Cout * Cin;
            FX_TAKES(c, "1x1 as batched slab GEMM (glk)");
            if (B == 1) return glk::run(c, pp, false, true, Cout, Cin, L, g, x, dw, nullptr, 0);
            float* part = (float*)(ws ? ws : c->get_scratch(need));
            if (!part) return FX_ERR_OOM;
            if (int rc = glk::run(c, pp, false, true, Cout, Cin, L, g, x, part, nullptr, 0, B, Cout * L, Cin * L, n)) return rc;
            return launch_splitk_reduce<T>(c, part, dw, n, (int)B);
        }
        const wgp::Plan pl = patch_plan<T>(c, d, mode);
        if (pl.ok && aligned16(x, g) && aligned16(ws, ws)) {
            float* part = (float*)(ws ? ws : c->get_scratch(need));
            if (!part) return FX_ERR_OOM;
            FX_TAKES(c, pl.segw ? "LDS patch, row segments (wgp)" : "LDS patch (wgp)");
            return wgp::run(c, pl, x, g, dw, part, Cin, H, W, Cout, sh, sw, ph, pw, d.oh, d.ow);
        }
    }
    if constexpr (sizeof(T) == 8) {
        if (mode == 0 && !generic_only()) {
            const cim::WPlan ip = cim::wgrad_plan(c->num_cus, d.B, d.Cin, d.H, d.W, d.Cout, d.kh, d.kw, d.sh, d.sw, d.ph, d.pw);
            if (ip.ok && aligned16(x, g) && aligned16(ws, ws)) {
                double* part = (double*)(ws ? ws : c->get_scratch(need));
                if (!part) return FX_ERR_OOM;
                return FX_TAKES(c, "image layer, row bands (cim)"), cim::run_wgrad(c, ip, x, g, dw, part, Cin, H, Cout);
            }
        }
        const wgd2::Plan q2 = patch64_s2_plan<T>(c, d, mode);
        if (q2.ok && aligned16(x, g) && aligned16(ws, ws)) {
            double* part = (double*)(ws ? ws : c->get_scratch(need));
            if (!part) return FX_ERR_OOM;
            return FX_TAKES(c, "stride-2 patch (wgd2)"), wgd2::run(c, q2, x, g, dw, part, Cin, H, Cout, ph, d.oh);
        }
        const wgd::Plan pd = patch64_plan<T>(c, d, mode);
        if (pd.ok && aligned16(x, g) && aligned16(ws, ws)) {
            double* part = (double*)(ws ? ws : c->get_scratch(need));
            if (!part) return FX_ERR_OOM;
            return FX_TAKES(c, "LDS patch (wgd)"), wgd::run(c, pd, x, g, dw, part, Cin, H, W, Cout, sh, ph, pw, d.oh, d.ow);
        }
    }
    FX_TAKES(c, mode == 0 ? "implicit GEMM" : "implicit GEMM (CPU-literal mode)");
    if (d.Cout > 64 && d.Cin * d.kh * d.kw > 64) return wgrad_tile<T, TileM128>(c, x, g, dw, d, mode, ws);
    if (d.Cout <= 32 && d.Cin * d.kh * d.kw <= 32) return wgrad_tile<T, TileTiny>(c, x, g, dw, d, mode, ws);
    return wgrad_tile<T, TileSmall>(c, x, g, dw, d, mode, ws);
}

// ---- backward of conv + ReLU from the UNMASKED upstream gradient --------------------------------------------------------
// The layer's ReLU gradient g * (act > 0) is applied while the consumer kernels stage g, and the weight-gradient kernel
// also leaves the bias gradient (the sums of the masked g per output channel): no masked copy of g is written or re-read
// and the separate mask + bias pass (fx_relu_bwd_bias_grad) disappears.  Kernels: the image-layer weight gradient
// (conv_smallc.hpp) and the stride-2 pair (wgrad_patch_s2.hpp, dgrad_patch_s2.hpp), f32.
template <typename T>
bool bwd_relu_supported(int num_cus, int kind, const Dims& d) {
    if constexpr (sizeof(T) == 4) {
        if (generic_only() || d.B > d.bc) return false;
        if (kind == FX_CONV_WGRAD) {
            if (csc::make_plan(num_cus, true, d.B, d.Cin, d.H, d.W, d.Cout, d.kh, d.kw, d.sh, d.sw, d.ph, d.pw, d.oh, d.ow).ok) return true;
            return wg2::make_plan(num_cus, d.B, d.Cin, d.H, d.W, d.Cout, d.kh, d.kw, d.sh, d.sw, d.ph, d.pw, d.oh, d.ow).ok;
        }
        if (kind == FX_CONV_DGRAD)
            return !dgrad_small_cin_ok<T>(d) && dg2::make_plan(d.B, d.Cin, d.H, d.W, d.Cout, d.kh, d.kw, d.sh, d.sw, d.ph, d.pw, d.oh, d.ow).ok;
    } else {
        if (generic_only() || d.B > d.bc) return false;
        if (kind == FX_CONV_WGRAD) {
            if (cim::wgrad_plan(num_cus, d.B, d.Cin, d.H, d.W, d.Cout, d.kh, d.kw, d.sh, d.sw, d.ph, d.pw).ok) return true;
            return wgd2::make_plan(num_cus, d.B, d.Cin, d.H, d.W, d.Cout, d.kh, d.kw, d.sh, d.sw, d.ph, d.pw, d.oh, d.ow).ok;
        }
        if (kind == FX_CONV_DGRAD)
            return !dgrad_small_cin_ok<T>(d) && dgd2::make_plan(d.B, d.Cin, d.H, d.W, d.Cout, d.kh, d.kw, d.sh, d.sw, d.ph, d.pw, d.oh, d.ow).ok;
    }
    return false;
}

template <typename T>
int conv_wgrad_relu_bias(fx_ctx* c, const T* x, const T* g, const T* act, T* dw, T* db, i64 B, i64 Cin, i64 H, i64 W, i64 Cout, i64 kh,
                         i64 kw, i64 sh, i64 sw, i64 ph, i64 pw, void* ws, i64 ws_bytes) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(x && g && act && dw && db, "fx_conv2d_wgrad_relu_bias: null pointer");
    Dims d;
    if (int rc = check_dims<T>(d, B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, "fx_conv2d_wgrad_relu_bias")) return rc;
    if constexpr (sizeof(T) == 4) {
        if (bwd_relu_supported<T>(c->num_cus, FX_CONV_WGRAD, d) && aligned16(x, g) && aligned16(act, ws)) {
            const i64 need = wgrad_ws_bytes<T>(c, d, 0);
            FX_REQUIRE(ws == nullptr || ws_bytes >= need, "fx_conv2d_wgrad_relu_bias: workspace of %lld bytes is smaller than the %lld needed",
                       (long long)ws_bytes, (long long)need);
            std::lock_guard<std::mutex> lk(c->launch_mutex);
            const csc::Plan sp = smallc_plan<T>(c, d, true);
            if (sp.ok) {
                float* part = nullptr;
                if (sp.splits > 1) {
                    part = (float*)(ws ? ws : c->get_scratch(need));
                    if (!part) return FX_ERR_OOM;
                }
                FX_TAKES(c, sp.rb ? "image layer, row bands (csc), ReLU mask and bias sums inside" : "image layer, tiles (csc), ReLU mask and bias sums inside");
                return csc::run_wgrad(c, sp, x, g, dw, part, Cin, H, W, Cout, d.oh, d.ow, sh, sw, ph, pw, act, db);
            }
            const wg2::Plan p2 = patch_s2_plan<T>(c, d, 0);
            if (p2.ok) {
                float* part = (float*)(ws ? ws : c->get_scratch(need));
                if (!part) return FX_ERR_OOM;
                return FX_TAKES(c, "stride-2 patch (wg2), ReLU mask and bias sums inside"), wg2::run(c, p2, x, g, dw, part, Cin, H, Cout, ph, d.oh, act, db);
            }
        }
    } else {
        if (bwd_relu_supported<T>(c->num_cus, FX_CONV_WGRAD, d) && aligned16(x, g) && aligned16(act, ws)) {
            const i64 need = wgrad_ws_bytes<T>(c, d, 0);
            FX_REQUIRE(ws == nullptr || ws_bytes >= need, "fx_conv2d_wgrad_relu_bias: workspace of %lld bytes is smaller than the %lld needed",
                       (long long)ws_bytes, (long long)need);
            std::lock_guard<std::mutex> lk(c->launch_mutex);
            double* part = (double*)(ws ? ws : c->get_scratch(need));
            if (!part) return FX_ERR_OOM;
            const cim::WPlan ip = cim::wgrad_plan(c->num_cus, d.B, d.Cin, d.H, d.W, d.Cout, d.kh, d.kw, d.sh, d.sw, d.ph, d.pw);
            if (ip.ok) return FX_TAKES(c, "image layer, row bands (cim), ReLU mask and bias sums inside"), cim::run_wgrad(c, ip, x, g, dw, part, Cin, H, Cout, act, db);
            const wgd2::Plan q2 = patch64_s2_plan<T>(c, d, 0);
            if (q2.ok) return FX_TAKES(c, "stride-2 patch (wgd2), ReLU mask and bias sums inside"), wgd2::run(c, q2, x, g, dw, part, Cin, H, Cout, ph, d.oh, act, db);
        }
    }
    fx::set_error("fx_conv2d_wgrad_relu_bias: no fused kernel for this shape, dtype or alignment (ask fx_conv2d_bwd_relu_supported; use "
                  "fx_relu_bwd_bias_grad + fx_conv2d_wgrad)");
    return FX_ERR_UNSUPPORTED;
}

template <typename T>
int conv_dgrad_relu(fx_ctx* c, const T* g, const T* act, const T* w, T* dx, i64 B, i64 Cin, i64 H, i64 W, i64 Cout, i64 kh, i64 kw, i64 sh,
                    i64 sw, i64 ph, i64 pw) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(g && act && w && dx, "fx_conv2d_dgrad_relu: null pointer");
    Dims d;
    if (int rc = check_dims<T>(d, B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, "fx_conv2d_dgrad_relu")) return rc;
    if constexpr (sizeof(T) == 4) {
        if (bwd_relu_supported<T>(c->num_cus, FX_CONV_DGRAD, d) && aligned16(g, w) && aligned16(dx, act)) {
            std::lock_guard<std::mutex> lk(c->launch_mutex);
            const dg2::Plan p2 = dg2::make_plan(d.B, d.Cin, d.H, d.W, d.Cout, d.kh, d.kw, d.sh, d.sw, d.ph, d.pw, d.oh, d.ow);
            return FX_TAKES(c, "stride-2 patch (dg2), ReLU mask inside"), dg2::run(c, p2, g, w, dx, B, Cin, Cout, d.oh, act);
        }
    } else {
        if (bwd_relu_supported<T>(c->num_cus, FX_CONV_DGRAD, d) && aligned16(g, w) && aligned16(dx, act)) {
            std::lock_guard<std::mutex> lk(c->launch_mutex);
            const dgd2::Plan p2 = dgd2::make_plan(d.B, d.Cin, d.H, d.W, d.Cout, d.kh, d.kw, d.sh, d.sw, d.ph, d.pw, d.oh, d.ow);
            return FX_TAKES(c, "stride-2 patch (dgd2), ReLU mask inside"), dgd2::run(c, p2, g, w, dx, B, Cin, Cout, d.oh, act);
        }
    }
    fx::set_error("fx_conv2d_dgrad_relu: no fused kernel for this shape, dtype or alignment (ask fx_conv2d_bwd_relu_supported; use "
                  "fx_relu_bwd + fx_conv2d_dgrad)");
    return FX_ERR_UNSUPPORTED;
}

}  // namespace

extern "C" const char* fx_conv2d_last_path(fx_ctx* c) { return c ? c->last_conv_path : ""; }

extern "C" int fx_conv2d_bwd_relu_supported(fx_ctx* c, int kind, int dtype, int64_t B, int64_t Cin, int64_t H, int64_t W, int64_t Cout,
                                            int64_t kh, int64_t kw, int64_t sh, int64_t sw, int64_t ph, int64_t pw) {
    Dims d;
    if (dtype == FX_F64) {
        if (check_dims<double>(d, B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, "fx_conv2d_bwd_relu_supported")) return 0;
        return bwd_relu_supported<double>(c ? c->num_cus : 256, kind, d) ? 1 : 0;
    }
    if (dtype != FX_F32 || check_dims<float>(d, B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, "fx_conv2d_bwd_relu_supported")) return 0;
    return bwd_relu_supported<float>(c ? c->num_cus : 256, kind, d) ? 1 : 0;
}

extern "C" int64_t fx_conv2d_workspace_bytes(int kind, int dtype, int mode, int64_t B, int64_t Cin, int64_t H, int64_t W,
                                             int64_t Cout, int64_t kh, int64_t kw, int64_t sh, int64_t sw, int64_t ph, int64_t pw) {
    Dims d;
    if (dtype == FX_F64 ? check_dims<double>(d, B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, "fx_conv2d_workspace_bytes")
                        : check_dims<float>(d, B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, "fx_conv2d_workspace_bytes"))
        return -1;
    auto need_of = [&](const Dims& q) -> i64 {
        if (kind == FX_CONV_FWD) return dtype == FX_F64 ? fwd_ws_bytes<double>(nullptr, q) : fwd_ws_bytes<float>(nullptr, q);
        if (kind == FX_CONV_DGRAD) return dtype == FX_F64 ? dgrad_ws_bytes<double>(nullptr, q, mode) : dgrad_ws_bytes<float>(nullptr, q, mode);
        return dtype == FX_F64 ? wgrad_ws_bytes<double>(nullptr, q, mode) : wgrad_ws_bytes<float>(nullptr, q, mode);
    };
    if (kind != FX_CONV_FWD && kind != FX_CONV_DGRAD && kind != FX_CONV_WGRAD) {
        fx::set_error("fx_conv2d_workspace_bytes: unknown kind %d", kind);
        return -1;
    }
    if (d.B <= d.bc) return need_of(d);
    // a batch that runs as slices: the largest need of a full slice and of the remainder
    Dims q = d;
    q.B = d.bc;
    i64 need = need_of(q);
    if (d.B % d.bc) {
        q.B = q.bc = d.B % d.bc;
        need = std::max(need, need_of(q));
    }
    return need;
}

// Pays the tile-shape timing of fx_conv2d_fwd / fx_conv2d_dgrad up front, on temporary zero-filled tensors of the layer's
// shape (allocated and released here; this entry point synchronises).
extern "C" int fx_conv2d_tune_f32(fx_ctx* c, int kind, int64_t B, int64_t Cin, int64_t H, int64_t W, int64_t Cout, int64_t kh,
                                  int64_t kw, int64_t sh, int64_t sw, int64_t ph, int64_t pw, int with_bias, int act) {
    FX_CHECK_CTX(c);
    FX_NOT_RECORDING(c, "fx_conv2d_tune");
    FX_REQUIRE(kind == FX_CONV_FWD || kind == FX_CONV_DGRAD || kind == FX_CONV_WGRAD, "fx_conv2d_tune: unknown kind %d", kind);
    FX_REQUIRE(act == 0 || act == 1, "fx_conv2d_tune: act must be 0 (none) or 1 (relu)");
    Dims d;
    if (int rc = check_dims<float>(d, B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, "fx_conv2d_tune")) return rc;
    if (kind == FX_CONV_WGRAD) return FX_OK;  // the weight-gradient kernels take their shape from the cost model alone
    const i64 nb = std::min(d.B, d.bc);       // a batch that runs as slices is timed at the slice size
    const i64 nx = nb * Cin * H * W, ny = nb * Cout * d.oh * d.ow, nw = Cout * Cin * kh * kw;
    float *x = nullptr, *y = nullptr, *w = nullptr, *bias = nullptr;
    auto release = [&] {
        (void)hipStreamSynchronize(c->stream);
        for (float* p : {x, y, w, bias})
            if (p) (void)hipFree(p);
    };
    hipError_t e = hipMalloc((void**)&x, (size_t)nx * 4);
    if (e == hipSuccess) e = hipMalloc((void**)&y, (size_t)ny * 4);
    if (e == hipSuccess) e = hipMalloc((void**)&w, (size_t)nw * 4);
    if (e == hipSuccess && with_bias) e = hipMalloc((void**)&bias, (size_t)Cout * 4);
    if (e == hipSuccess) e = hipMemsetAsync(x, 0, (size_t)nx * 4, c->stream);
    if (e == hipSuccess) e = hipMemsetAsync(y, 0, (size_t)ny * 4, c->stream);
    if (e == hipSuccess) e = hipMemsetAsync(w, 0, (size_t)nw * 4, c->stream);
    if (e == hipSuccess && bias) e = hipMemsetAsync(bias, 0, (size_t)Cout * 4, c->stream);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        release();
        fx::set_error("fx_conv2d_tune: temporary tensors: %s", hipGetErrorString(e));
        return e == hipErrorOutOfMemory ? FX_ERR_OOM : FX_ERR_HIP;
    }
    c->conv_retune = true;
    int rc;
    if (kind == FX_CONV_FWD) rc = conv_fwd<float>(c, x, w, y, nb, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, nullptr, 0, bias, act);
    else rc = conv_dgrad<float>(c, y, w, x, nb, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, 0, nullptr, 0);
    c->conv_retune = false;
    release();
    return rc;
}

#define FX_DEFINE_CONV(T, S)                                                                                           \
    extern "C" int fx_conv2d_fwd_##S(fx_ctx* c, const T* x, const T* w, T* y, int64_t B, int64_t Cin, int64_t H, int64_t W, \
                                     int64_t Cout, int64_t kh, int64_t kw, int64_t sh, int64_t sw, int64_t ph, int64_t pw,  \
                                     void* ws, int64_t ws_bytes) {                                                     \
        return conv_fwd<T>(c, x, w, y, B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, ws, ws_bytes);                      \
    }                                                                                                                  \
    extern "C" int fx_conv2d_fwd_bias_act_##S(fx_ctx* c, const T* x, const T* w, const T* bias, T* y, int64_t B, int64_t Cin,  \
                                              int64_t H, int64_t W, int64_t Cout, int64_t kh, int64_t kw, int64_t sh,     \
                                              int64_t sw, int64_t ph, int64_t pw, int act, void* ws, int64_t ws_bytes) { \
        FX_REQUIRE(bias != nullptr, "fx_conv2d_fwd_bias_act: null bias");                                              \
        FX_REQUIRE(act == 0 || act == 1, "fx_conv2d_fwd_bias_act: act must be 0 (none) or 1 (relu)");                  \
        return conv_fwd<T>(c, x, w, y, B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, ws, ws_bytes, bias, act);           \
    }                                                                                                                  \
    extern "C" int fx_conv2d_dgrad_##S(fx_ctx* c, const T* g, const T* w, T* dx, int64_t B, int64_t Cin, int64_t H, int64_t W, \
                                       int64_t Cout, int64_t kh, int64_t kw, int64_t sh, int64_t sw, int64_t ph, int64_t pw,   \
                                       int mode, void* ws, int64_t ws_bytes) {                                         \
        return conv_dgrad<T>(c, g, w, dx, B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, mode, ws, ws_bytes);             \
    }                                                                                                                  \
    extern "C" int fx_conv2d_wgrad_##S(fx_ctx* c, const T* x, const T* g, T* dw, int64_t B, int64_t Cin, int64_t H, int64_t W, \
                                       int64_t Cout, int64_t kh, int64_t kw, int64_t sh, int64_t sw, int64_t ph, int64_t pw,   \
                                       int mode, void* ws, int64_t ws_bytes) {                                         \
        return conv_wgrad<T>(c, x, g, dw, B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, mode, ws, ws_bytes);             \
    }                                                                                                                  \
    extern "C" int fx_conv2d_wgrad_relu_bias_##S(fx_ctx* c, const T* x, const T* g, const T* act, T* dw, T* db, int64_t B,   \
                                                 int64_t Cin, int64_t H, int64_t W, int64_t Cout, int64_t kh, int64_t kw,  \
                                                 int64_t sh, int64_t sw, int64_t ph, int64_t pw, void* ws, int64_t ws_bytes) { \
        return conv_wgrad_relu_bias<T>(c, x, g, act, dw, db, B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, ws, ws_bytes); \
    }                                                                                                                  \
    extern "C" int fx_conv2d_dgrad_relu_##S(fx_ctx* c, const T* g, const T* act, const T* w, T* dx, int64_t B, int64_t Cin,   \
                                            int64_t H, int64_t W, int64_t Cout, int64_t kh, int64_t kw, int64_t sh,   \
                                            int64_t sw, int64_t ph, int64_t pw) {                                      \
        return conv_dgrad_relu<T>(c, g, act, w, dx, B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw);                       \
    }

FX_DEFINE_CONV(float, f32)
FX_DEFINE_CONV(double, f64)
