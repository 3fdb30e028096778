// Implicit-GEMM core for gfx950: one LDS-staged, MFMA-fed tile kernel shared by the plain GEMM and the three
// convolution passes.  C[M,N] = sum_k A(m,k) * B(k,n), where A, B and the store of C are small policy objects:
//   - "loaders" fetch one BK-deep slab of an operand from global memory into registers (doing the im2col /
//     col2im address arithmetic on the fly for convolutions, so no column matrix is ever materialised) and
//     write it to LDS as [k][m] / [k][n];
//   - the main loop reads MFMA operands straight from those LDS rows (lane l reads row k0 + l/BLK, column
//     l%BLK: consecutive lanes hit consecutive banks) and issues v_mfma_f32_32x32x2_f32 or
//     v_mfma_f64_16x16x4_f64;
//   - the epilogue scatters accumulators to their final layout (row-major matrix, NCHW tensor, or split-K
//     partial).
// Loaders are branch-free: an element outside the operand (padding ring, ragged tile edge, K tail) is fetched
// from a clamped in-range address and replaced by zero afterwards, so all global loads of a slab sit in one basic
// block and can be scheduled behind the MFMA stream.  Addresses are a wave-uniform 64-bit base plus a 32-bit byte
// offset per lane (hosts check that the addressed tensor is below 2 GiB and M, N, K below 2^31).
// Global loads for slab i+1 are issued before the MFMA loop of slab i; LDS is double-buffered so there is one
// barrier per slab; several blocks are resident per CU so one block's barrier overlaps another block's MFMAs.
#pragma once
#include <algorithm>
#include <climits>

#include "common.hpp"

#ifndef FX_KPAD
#define FX_KPAD 2
#endif

namespace igemm {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef double f64x4 __attribute__((ext_vector_type(4)));

// Division by a runtime constant as multiply-high + shift (exact for all 32-bit n).
struct FastDiv {
    uint32_t d, m, s;
    FastDiv() : d(1), m(1), s(0) {}
    explicit FastDiv(uint32_t d_) : d(d_ ? d_ : 1) {  // a zero divisor (an empty extent that is never indexed) acts as 1
        s = 0;
        while ((1ull << s) < d) ++s;
        m = (uint32_t)((((1ull << 32) * ((1ull << s) - d)) / d) + 1);
    }
    __device__ __forceinline__ uint32_t div(uint32_t n) const { return (uint32_t)(((uint64_t)__umulhi(n, m) + n) >> s); }
};

// Load from a wave-uniform base plus a 32-bit unsigned byte offset.
template <typename T> __device__ __forceinline__ T ldg(const T* base, uint32_t byteoff) {
    return *reinterpret_cast<const T*>(reinterpret_cast<const char*>(base) + byteoff);
}

template <typename T> struct Mfma;
template <> struct Mfma<float> {
    static constexpr int BLK = 32, KSTEP = 2, NACC = 16;
    typedef f32x16 Acc;
    static __device__ __forceinline__ Acc mma(float a, float b, Acc c) { return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0); }
    // accumulator element e of lane l holds C[row(e,l)][l % 32]
    static __device__ __forceinline__ int row(int e, int lane) { return 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3); }
};
template <> struct Mfma<double> {
    static constexpr int BLK = 16, KSTEP = 4, NACC = 4;
    typedef f64x4 Acc;
    static __device__ __forceinline__ Acc mma(double a, double b, Acc c) { return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0); }
    // accumulator element e of lane l holds C[4*e + l/16][l % 16]
    static __device__ __forceinline__ int row(int e, int lane) { return 4 * e + (lane >> 4); }
};

// Block tile BM x BN x BK computed by (BM/WM) x (BN/WN) waves, each owning a WM x WN sub-tile.
// 16-byte load from global memory at a wave-uniform base plus a 32-bit byte offset (never a FLAT access, so it
// does not tie up the LDS counter that the MFMA loop waits on).
__device__ __forceinline__ float4 ldg4(const float* base, uint32_t byteoff) {
    typedef __attribute__((address_space(1))) const char gchar;
    typedef float v4 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(1))) const v4 gv4;
    const v4 v = *(gv4*)((gchar*)base + byteoff);
    return make_float4(v.x, v.y, v.z, v.w);
}

template <int BM_, int BN_, int BK_, int WM_, int WN_> struct Tile {
    static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_;
    static constexpr int WAVES_M = BM / WM, WAVES_N = BN / WN;
    static constexpr int NT = WAVES_M * WAVES_N * 64;
};

// Which (k, mn) element of the slab register i of thread `tid` holds.
//  KMAJOR (operand contiguous along k):   k = tid % BK (fixed per thread), mn = tid / BK + i * (NT / BK)
//  else   (operand contiguous along m/n): mn = tid % BMN (fixed per thread), k = tid / BMN + i * (NT / BMN)
template <int BMN, int BK, int NT, bool KMAJOR> struct SlabMap {
    static constexpr int CNT = BMN * BK / NT;
    static constexpr int STEP = KMAJOR ? NT / BK : NT / BMN;
    static constexpr int LD = KMAJOR ? BMN + FX_KPAD : BMN;  // LDS row pitch; the pad spreads the transposing writes over banks
    static_assert(BMN * BK % NT == 0, "slab must divide evenly over the block");
    static_assert(KMAJOR ? (NT % BK == 0) : (NT % BMN == 0 && BMN % 64 == 0), "unsupported tile/thread shape");
    static __device__ __forceinline__ int k_of(int tid, int i) { return KMAJOR ? tid % BK : tid / BMN + i * STEP; }
    static __device__ __forceinline__ int mn_of(int tid, int i) { return KMAJOR ? tid / BK + i * STEP : tid % BMN; }
    template <typename T> static __device__ __forceinline__ void store(T* lds, const T (&r)[CNT], int tid) {
#pragma unroll
        for (int i = 0; i < CNT; ++i) lds[k_of(tid, i) * LD + mn_of(tid, i)] = r[i];
    }
};

// ---- plain matrix operand --------------------------------------------------------------------------------
// KMAJOR: element (mn, k) at p[mn * ld + k];  otherwise at p[k * ld + mn].
template <typename T, bool KMAJOR_> struct MatLoader {
    static constexpr bool KMAJOR = KMAJOR_;
    const T* p;
    i64 ld;
    int MN;
    template <int BMN, int BK, int NT> struct Dev {
        typedef SlabMap<BMN, BK, NT, KMAJOR_> Map;
        const T* base;          // wave-uniform: first row (KMAJOR) / first column (otherwise) of this block's tile
        i64 ld;
        uint32_t off[KMAJOR_ ? Map::CNT : 1];  // byte offsets from base (rows clamped into the matrix)
        uint32_t okmask;        // bit i: register i addresses a row/column inside the matrix
        uint32_t live;          // validity of the slab in flight, consumed by mask()
        int klane, krow;
        __device__ __forceinline__ Dev(const MatLoader& L, int origin, int tid) : ld(L.ld) {
            okmask = 0;
            if (KMAJOR_) {
                base = L.p + (i64)origin * L.ld;
                klane = tid % BK;
                krow = 0;
#pragma unroll
                for (int i = 0; i < Map::CNT; ++i) {
                    const int r = Map::mn_of(tid, i);
                    const bool ok = origin + r < L.MN;
                    okmask |= ok ? (1u << i) : 0u;
                    off[i] = (uint32_t)(((ok ? r : 0) * (uint32_t)L.ld + klane) * sizeof(T));
                }
            } else {
                base = L.p + origin;
                const int r = tid % BMN;
                const bool ok = origin + r < L.MN;
                okmask = ok ? ~0u : 0u;
                off[0] = (uint32_t)((ok ? r : 0) * sizeof(T));
                klane = 0;
                krow = __builtin_amdgcn_readfirstlane(tid / BMN);
            }
        }
        // load() only issues the global loads (from clamped addresses); mask() zeroes what lay outside the operand.
        // The kernel calls mask() after the MFMA loop, so the loads stay in flight behind the matrix work.
        __device__ __forceinline__ void load(int k0, int kend, T (&r)[Map::CNT]) {
            if (KMAJOR_) {
                const bool kok = k0 + klane < kend;
                live = kok ? okmask : 0u;
                const T* b = base + k0;  // uniform
#pragma unroll
                for (int i = 0; i < Map::CNT; ++i) r[i] = ldg(b, kok ? off[i] : 0u);
            } else {
                live = 0;
#pragma unroll
                for (int i = 0; i < Map::CNT; ++i) {
                    const int k = k0 + krow + i * Map::STEP;       // uniform
                    const int kc = min(k, kend - 1);               // clamped row stays inside the split
                    r[i] = ldg(base + (i64)kc * ld, off[0]);
                    live |= (k < kend && okmask) ? (1u << i) : 0u;
                }
            }
        }
        __device__ __forceinline__ void mask(T (&r)[Map::CNT]) const {
#pragma unroll
            for (int i = 0; i < Map::CNT; ++i) r[i] = ((live >> i) & 1u) ? r[i] : T(0);
        }
    };
};

// ---- convolution geometry shared by the conv loaders -------------------------------------------------------
struct ConvShape {
    int B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, oh, ow;
    FastDiv div_L, div_ow, div_KK, div_kw, div_HW, div_W, div_sh, div_sw, div_Cin, div_Cout;
};

// Forward B operand: B(k, n = (b,oy,ox)) = x[b, c, oy*sh + ky - ph, ox*sw + kx - pw] (0 outside the image).
// Contiguous along n.  The pixel of a thread is fixed for the whole kernel; k is wave-uniform.
//  FAST  : k = (ky*kw + kx)*Cin + c with Cin % BK == 0 (the host permutes the weights to match): all BK rows of a
//          slab share (ky,kx), so the bounds test is done once per slab and rows differ by a uniform H*W stride.
//  !FAST : k = (c*kh + ky)*kw + kx as in the reference im2col; every row decodes its own (c,ky,kx).
template <typename T, bool FAST> struct ConvFwdB {
    static constexpr bool KMAJOR = false;
    const T* x;
    ConvShape s;
    int N;
    template <int BMN, int BK, int NT> struct Dev {
        typedef SlabMap<BMN, BK, NT, false> Map;
        const T* x; const ConvShape& s; int pix, iy0, ix0, krow; bool ok; uint32_t live;
        __device__ __forceinline__ Dev(const ConvFwdB& L, int origin, int tid) : x(L.x), s(L.s) {
            const int n = origin + tid % BMN;
            ok = n < L.N;
            const uint32_t nn = ok ? n : 0;
            const uint32_t b = s.div_L.div(nn), l = nn - b * (s.oh * s.ow);
            const uint32_t oy = s.div_ow.div(l), ox = l - oy * s.ow;
            iy0 = (int)oy * s.sh - s.ph;
            ix0 = (int)ox * s.sw - s.pw;
            pix = (((int)b * s.Cin * s.H + iy0) * s.W + ix0) * (int)sizeof(T);  // signed byte offset of tap (c=0,ky=0,kx=0)
            krow = __builtin_amdgcn_readfirstlane(tid / BMN);
        }
        __device__ __forceinline__ void load(int k0, int kend, T (&r)[Map::CNT]) {
            const int HW = s.H * s.W;
            if (FAST) {
                const uint32_t kyx = s.div_Cin.div(k0), c0 = k0 - kyx * s.Cin;
                const uint32_t ky = s.div_kw.div(kyx), kx = kyx - ky * s.kw;
                const bool in = ok && (unsigned)(iy0 + (int)ky) < (unsigned)s.H && (unsigned)(ix0 + (int)kx) < (unsigned)s.W;
                live = in ? ~0u : 0u;
                const int uni = (((int)c0 + krow) * HW + (int)ky * s.W + (int)kx) * (int)sizeof(T);
                const uint32_t v = in ? (uint32_t)(pix + uni) : 0u;
#pragma unroll
                for (int i = 0; i < Map::CNT; ++i) r[i] = ldg(x, v + (uint32_t)(i * Map::STEP * HW * (int)sizeof(T)));
            } else {
                const int KK = s.kh * s.kw;
                live = 0;
#pragma unroll
                for (int i = 0; i < Map::CNT; ++i) {
                    const int k = k0 + krow + i * Map::STEP;
                    const uint32_t c = s.div_KK.div(k), rr = k - c * KK;
                    const uint32_t ky = s.div_kw.div(rr), kx = rr - ky * s.kw;
                    const bool in = ok && k < kend && (unsigned)(iy0 + (int)ky) < (unsigned)s.H && (unsigned)(ix0 + (int)kx) < (unsigned)s.W;
                    live |= in ? (1u << i) : 0u;
                    const int uni = ((int)c * HW + (int)ky * s.W + (int)kx) * (int)sizeof(T);
                    r[i] = ldg(x, in ? (uint32_t)(pix + uni) : 0u);
                }
            }
        }
        __device__ __forceinline__ void mask(T (&r)[Map::CNT]) const {
#pragma unroll
            for (int i = 0; i < Map::CNT; ++i) r[i] = ((live >> i) & 1u) ? r[i] : T(0);
        }
    };
};

// Data-gradient B operand: B(k, n = (b,y,x)) = g[b, oc, (y+ph-ky)/sh, (x+pw-kx)/sw] when both quotients are exact
// and inside the output plane, else 0.  This is the gather form of col2im: every input pixel is owned by exactly
// one accumulator, so there are no races and no atomics.
//  FAST  : k = (ky*kw + kx)*Cout + oc with Cout % BK == 0;  !FAST : k = (oc*kh + ky)*kw + kx.
template <typename T, bool FAST> struct ConvDgradB {
    static constexpr bool KMAJOR = false;
    const T* g;
    ConvShape s;
    int N;  // B*H*W
    template <int BMN, int BK, int NT> struct Dev {
        typedef SlabMap<BMN, BK, NT, false> Map;
        const T* g; const ConvShape& s; int img, yp, xp, krow; bool ok; uint32_t live;
        __device__ __forceinline__ Dev(const ConvDgradB& L, int origin, int tid) : g(L.g), s(L.s) {
            const int n = origin + tid % BMN;
            ok = n < L.N;
            const uint32_t nn = ok ? n : 0;
            const uint32_t b = s.div_HW.div(nn), p = nn - b * (s.H * s.W);
            const uint32_t y = s.div_W.div(p), x = p - y * s.W;
            img = (int)b * s.Cout * s.oh * s.ow * (int)sizeof(T);
            yp = (int)y + s.ph;
            xp = (int)x + s.pw;
            krow = __builtin_amdgcn_readfirstlane(tid / BMN);
        }
        // byte offset of g[b, 0, cy, cx] for tap (ky,kx); `in` false when the tap does not reach the output plane
        __device__ __forceinline__ int tap(int ky, int kx, bool& in) const {
            const int ty = yp - ky, tx = xp - kx;
            in = ok && ty >= 0 && tx >= 0;
            int cy = ty, cx = tx;
            if (!(s.sh == 1 && s.sw == 1)) {
                cy = (int)s.div_sh.div(in ? (uint32_t)ty : 0u);
                cx = (int)s.div_sw.div(in ? (uint32_t)tx : 0u);
                in = in && cy * s.sh == ty && cx * s.sw == tx;
            }
            in = in && cy < s.oh && cx < s.ow;
            return img + (cy * s.ow + cx) * (int)sizeof(T);
        }
        __device__ __forceinline__ void load(int k0, int kend, T (&r)[Map::CNT]) {
            const int L = s.oh * s.ow;
            if (FAST) {
                const uint32_t kyx = s.div_Cout.div(k0), oc0 = k0 - kyx * s.Cout;
                const uint32_t ky = s.div_kw.div(kyx), kx = kyx - ky * s.kw;
                bool in;
                const int t = tap((int)ky, (int)kx, in);
                live = in ? ~0u : 0u;
                const uint32_t v = in ? (uint32_t)(t + ((int)oc0 + krow) * L * (int)sizeof(T)) : 0u;
#pragma unroll
                for (int i = 0; i < Map::CNT; ++i) r[i] = ldg(g, v + (uint32_t)(i * Map::STEP * L * (int)sizeof(T)));
            } else {
                const int KK = s.kh * s.kw;
                live = 0;
#pragma unroll
                for (int i = 0; i < Map::CNT; ++i) {
                    const int k = k0 + krow + i * Map::STEP;
                    const uint32_t oc = s.div_KK.div(k), rr = k - oc * KK;
                    const uint32_t ky = s.div_kw.div(rr), kx = rr - ky * s.kw;
                    bool in;
                    const int t = tap((int)ky, (int)kx, in);
                    in = in && k < kend;
                    live |= in ? (1u << i) : 0u;
                    r[i] = ldg(g, in ? (uint32_t)(t + (int)oc * L * (int)sizeof(T)) : 0u);
                }
            }
        }
        __device__ __forceinline__ void mask(T (&r)[Map::CNT]) const {
#pragma unroll
            for (int i = 0; i < Map::CNT; ++i) r[i] = ((live >> i) & 1u) ? r[i] : T(0);
        }
    };
};

// Weight-gradient A operand: A(m = oc, k = (b,l)) = g[(b*Cout + oc)*L + l].  Contiguous along k inside an image.
template <typename T> struct ConvWgradA {
    static constexpr bool KMAJOR = true;
    const T* g;
    ConvShape s;
    template <int BMN, int BK, int NT> struct Dev {
        typedef SlabMap<BMN, BK, NT, true> Map;
        const T* g; const ConvShape& s; int klane;
        uint32_t moff[Map::CNT];  // oc * L * sizeof(T), oc clamped into range
        uint32_t okmask, live;
        __device__ __forceinline__ Dev(const ConvWgradA& L, int origin, int tid) : g(L.g), s(L.s) {
            klane = tid % BK;
            okmask = 0;
            const int Lp = s.oh * s.ow;
#pragma unroll
            for (int i = 0; i < Map::CNT; ++i) {
                const int m = origin + Map::mn_of(tid, i);
                const bool ok = m < s.Cout;
                okmask |= ok ? (1u << i) : 0u;
                moff[i] = (uint32_t)((ok ? m : 0) * Lp * (int)sizeof(T));
            }
        }
        __device__ __forceinline__ void load(int k0, int kend, T (&r)[Map::CNT]) {
            const int k = k0 + klane;
            const bool kok = k < kend;
            live = kok ? okmask : 0u;
            const int L = s.oh * s.ow;
            const uint32_t kk = kok ? k : (uint32_t)k0;  // k0 < kend always
            const uint32_t b = s.div_L.div(kk), l = kk - b * L;
            const uint32_t v = (b * (uint32_t)s.Cout * L + l) * (uint32_t)sizeof(T);
#pragma unroll
            for (int i = 0; i < Map::CNT; ++i) r[i] = ldg(g, v + moff[i]);
        }
        __device__ __forceinline__ void mask(T (&r)[Map::CNT]) const {
#pragma unroll
            for (int i = 0; i < Map::CNT; ++i) r[i] = ((live >> i) & 1u) ? r[i] : T(0);
        }
    };
};

// Weight-gradient B operand: B(k = (b,oy,ox), n = (c,ky,kx)) = x[b, c, oy*sh+ky-ph, ox*sw+kx-pw] (0 outside):
// the im2col matrix read transposed.  The (c,ky,kx) of each register is fixed for the whole kernel and decoded once.
template <typename T> struct ConvWgradB {
    static constexpr bool KMAJOR = true;
    const T* x;
    ConvShape s;
    int N;  // Cin*kh*kw
    template <int BMN, int BK, int NT> struct Dev {
        typedef SlabMap<BMN, BK, NT, true> Map;
        const T* x; const ConvShape& s; int klane; uint32_t live;
        int off[Map::CNT];   // (c*H*W + (ky-ph)*W + (kx-pw)) * sizeof(T)
        int kyx[Map::CNT];   // (ky-ph) << 16 | ((kx-pw) & 0xffff); INT_MIN when the column is out of range
        __device__ __forceinline__ Dev(const ConvWgradB& L, int origin, int tid) : x(L.x), s(L.s) {
            klane = tid % BK;
            const int KK = s.kh * s.kw;
#pragma unroll
            for (int i = 0; i < Map::CNT; ++i) {
                const int n = origin + Map::mn_of(tid, i);
                if (n < L.N) {
                    const uint32_t c = s.div_KK.div(n), rr = n - c * KK;
                    const uint32_t ky = s.div_kw.div(rr), kx = rr - ky * s.kw;
                    const int dy = (int)ky - s.ph, dx = (int)kx - s.pw;
                    off[i] = (((int)c * s.H + dy) * s.W + dx) * (int)sizeof(T);
                    kyx[i] = (int)(((uint32_t)dy << 16) | ((uint32_t)dx & 0xffffu));
                } else {
                    off[i] = 0;
                    kyx[i] = INT_MIN;
                }
            }
        }
        __device__ __forceinline__ void load(int k0, int kend, T (&r)[Map::CNT]) {
            const int k = k0 + klane;
            const bool kok = k < kend;
            const uint32_t kk = kok ? k : (uint32_t)k0;
            const int L = s.oh * s.ow;
            const uint32_t b = s.div_L.div(kk), l = kk - b * L;
            const uint32_t oy = s.div_ow.div(l), ox = l - oy * s.ow;
            const int y0 = (int)oy * s.sh, x0 = (int)ox * s.sw;
            const int pix = (((int)b * s.Cin * s.H + y0) * s.W + x0) * (int)sizeof(T);
            live = 0;
#pragma unroll
            for (int i = 0; i < Map::CNT; ++i) {
                const int dy = kyx[i] >> 16, dx = (int)(short)(kyx[i] & 0xffff);
                const bool in = kok && kyx[i] != INT_MIN && (unsigned)(y0 + dy) < (unsigned)s.H && (unsigned)(x0 + dx) < (unsigned)s.W;
                live |= in ? (1u << i) : 0u;
                r[i] = ldg(x, in ? (uint32_t)(pix + off[i]) : 0u);
            }
        }
        __device__ __forceinline__ void mask(T (&r)[Map::CNT]) const {
#pragma unroll
            for (int i = 0; i < Map::CNT; ++i) r[i] = ((live >> i) & 1u) ? r[i] : T(0);
        }
    };
};

// ---- epilogues ---------------------------------------------------------------------------------------------
// An epilogue maps a column n to a base pointer (col) and stores row m at q[m * row_stride]; xform(m, n, v) is
// applied to every stored value: identity, or with BIAS (a compile-time switch, so that the plain kernels carry no
// trace of it) v + bias, then ReLU when relu != 0.
// Row-major matrix (also used for split-K partials: split z goes to p + z*split_stride).  bias is per column n.
template <typename T, bool BIAS = false> struct MatStore {
    T* p;
    i64 ld, split_stride;
    int M, N;
    const T* bias = nullptr;
    int relu = 0;
    __device__ __forceinline__ int rows() const { return M; }
    __device__ __forceinline__ int cols() const { return N; }
    __device__ __forceinline__ i64 row_stride() const { return ld; }
    __device__ __forceinline__ T* col(int n, int split) const { return p + (i64)split * split_stride + n; }
    __device__ __forceinline__ T xform(int, int n, T v) const {
        if constexpr (BIAS) {
            v = v + bias[n];
            if (relu) v = v > T(0) ? v : T(0);
        }
        return v;
    }
};
// NCHW tensor: row m = channel, column n = (b, l) -> p[(b*C + m)*L + l].
template <typename T, bool BIAS = false> struct NchwStore {  // bias is per row m (channel)
    T* p;
    int C, L, N;
    FastDiv div_L;
    const T* bias = nullptr;
    int relu = 0;
    __device__ __forceinline__ T xform(int m, int, T v) const {
        if constexpr (BIAS) {
            v = v + bias[m];
            if (relu) v = v > T(0) ? v : T(0);
        }
        return v;
    }
    __device__ __forceinline__ int rows() const { return C; }
    __device__ __forceinline__ int cols() const { return N; }
    __device__ __forceinline__ i64 row_stride() const { return L; }
    __device__ __forceinline__ T* col(int n, int) const {
        const uint32_t b = div_L.div(n), l = n - b * L;
        return p + (i64)b * C * L + l;
    }
};

// A strided sub-grid of an NCHW tensor [.., C, H, W]: column n = (b, yy, xx) over a [Hs, Ws] grid lands on pixel
// (y0 + yy*sy, x0 + xx*sx); row m = channel.
template <typename T> struct NchwSubgridStore {
    T* p;
    int C, H, W, Hs, Ws, y0, x0, sy, sx, N;
    FastDiv div_grid, div_ws;
    __device__ __forceinline__ T xform(int, int, T v) const { return v; }
    __device__ __forceinline__ int rows() const { return C; }
    __device__ __forceinline__ int cols() const { return N; }
    __device__ __forceinline__ i64 row_stride() const { return (i64)H * W; }
    __device__ __forceinline__ T* col(int n, int) const {
        const uint32_t b = div_grid.div(n), l = n - b * (Hs * Ws);
        const uint32_t yy = div_ws.div(l), xx = l - yy * Ws;
        return p + ((i64)b * C * H + (y0 + (int)yy * sy)) * W + (x0 + (int)xx * sx);
    }
};

// ---- the kernel -------------------------------------------------------------------------------------------
// grid (N tiles, M tiles, K splits).  Split z covers k in [z*kps, min(K, (z+1)*kps)), kps a multiple of BK.
// The tile program; (tile_n, tile_m, split) normally come from blockIdx.
template <typename T, class Cfg, class AL, class BL, class EP>
__device__ __forceinline__ void igemm_tile(const AL& al, const BL& bl, const EP& ep, int K, int kps, int tile_n, int tile_m, int split) {
    typedef Mfma<T> MF;
    constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, NT = Cfg::NT;
    constexpr int TM = Cfg::WM / MF::BLK, TN = Cfg::WN / MF::BLK;
    static_assert(Cfg::WM % MF::BLK == 0 && Cfg::WN % MF::BLK == 0 && BK % MF::KSTEP == 0, "tile must be a multiple of the MFMA block");
    typedef typename AL::template Dev<BM, BK, NT> ADev;
    typedef typename BL::template Dev<BN, BK, NT> BDev;
    typedef typename ADev::Map AMap;
    typedef typename BDev::Map BMap;

    // Two LDS stages: while the MFMA loop reads stage `cur`, the next slab (already in registers) is written to the
    // other stage, so one barrier per slab suffices.
    __shared__ T As[2][BK * AMap::LD];
    __shared__ T Bs[2][BK * BMap::LD];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int bm = tile_m * BM, bn = tile_n * BN;
    const int kbeg = split * kps, kend = min(K, kbeg + kps);
    const int wm0 = (wave / Cfg::WAVES_N) * Cfg::WM, wn0 = (wave % Cfg::WAVES_N) * Cfg::WN;

    ADev ad(al, bm, tid);
    BDev bd(bl, bn, tid);

    typename MF::Acc acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < MF::NACC; ++e) acc[i][j][e] = T(0);

    T ra[AMap::CNT], rb[BMap::CNT];
    ad.load(kbeg, kend, ra);
    bd.load(kbeg, kend, rb);
    ad.mask(ra);
    bd.mask(rb);
    AMap::store(As[0], ra, tid);
    BMap::store(Bs[0], rb, tid);
    __syncthreads();

    const int lrow = lane / MF::BLK, lcol = lane % MF::BLK;
    constexpr int STORE_AT = (BK / MF::KSTEP * 3 / 4) * MF::KSTEP;  // k-step at which the prefetched slab goes to LDS
    int cur = 0;
    for (int k0 = kbeg; k0 < kend; k0 += BK) {
        const bool more = k0 + BK < kend;
        if (more) {  // global loads for the next slab fly while this slab is multiplied
            ad.load(k0 + BK, kend, ra);
            bd.load(k0 + BK, kend, rb);
        }
        const T* Ac = As[cur] + lrow * AMap::LD + wm0 + lcol;
        const T* Bc = Bs[cur] + lrow * BMap::LD + wn0 + lcol;
#pragma unroll
        for (int kk = 0; kk < BK; kk += MF::KSTEP) {
            if (kk == STORE_AT && more) {
                // The next slab's loads were issued a half slab of MFMAs ago; writing them to the other LDS stage
                // here lets the LDS stores drain under the remaining MFMAs instead of after them.
                __builtin_amdgcn_sched_barrier(0);
                ad.mask(ra);
                bd.mask(rb);
                AMap::store(As[cur ^ 1], ra, tid);
                BMap::store(Bs[cur ^ 1], rb, tid);
                __builtin_amdgcn_sched_barrier(0);
            }
            T a[TM], b[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) a[i] = Ac[kk * AMap::LD + i * MF::BLK];
#pragma unroll
            for (int j = 0; j < TN; ++j) b[j] = Bc[kk * BMap::LD + j * MF::BLK];
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[i][j] = MF::mma(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
        cur ^= 1;
    }

    const int M = ep.rows(), N = ep.cols();
    const i64 rs = ep.row_stride();
    if (bm + BM <= M && bn + BN <= N) {  // interior tile: no edge tests
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int n = bn + wn0 + j * MF::BLK + lcol;
            T* q = ep.col(n, split) + (i64)(bm + wm0) * rs;
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int e = 0; e < MF::NACC; ++e) {
                    const int r = i * MF::BLK + MF::row(e, lane);
                    q[(i64)r * rs] = ep.xform(bm + wm0 + r, n, acc[i][j][e]);
                }
        }
    } else {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int n = bn + wn0 + j * MF::BLK + lcol;
            if (n < N) {
                T* q = ep.col(n, split);
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int e = 0; e < MF::NACC; ++e) {
                        const int m = bm + wm0 + i * MF::BLK + MF::row(e, lane);
                        if (m < M) q[(i64)m * rs] = ep.xform(m, n, acc[i][j][e]);
                    }
            }
        }
    }
}

template <typename T, class Cfg, class AL, class BL, class EP>
__global__ __launch_bounds__(Cfg::NT) void igemm_kernel(AL al, BL bl, EP ep, int K, int kps) {
    igemm_tile<T, Cfg, AL, BL, EP>(al, bl, ep, K, kps, blockIdx.x, blockIdx.y, blockIdx.z);
}

// Up to NP independent problems of one kind in a single launch (blockIdx.z picks the problem, no K split): used where
// one operator decomposes into a few small GEMMs that would each leave most of the chip idle.
template <class AL, class BL, class EP, int NP> struct MultiProblem {
    AL al[NP];
    BL bl[NP];
    EP ep[NP];
    int K[NP], kps[NP], tiles_n[NP], tiles_m[NP];
};
template <typename T, class Cfg, class AL, class BL, class EP, int NP>
__global__ __launch_bounds__(Cfg::NT) void igemm_multi_kernel(const MultiProblem<AL, BL, EP, NP> mp) {
    const int z = blockIdx.z;  // wave-uniform: the kernel arguments are read with scalar loads
    if ((int)blockIdx.x >= mp.tiles_n[z] || (int)blockIdx.y >= mp.tiles_m[z]) return;
    igemm_tile<T, Cfg, AL, BL, EP>(mp.al[z], mp.bl[z], mp.ep[z], mp.K[z], mp.kps[z], blockIdx.x, blockIdx.y, 0);
}

// Sums split-K partials in split order (deterministic) into the final buffer; 8 independent loads in flight.
// Optional epilogue of the sums below: + bias[column] (row-major [rows][ncols] outputs), then ReLU -- the operations of
// fx_bias_act in its order, so the bits are those of the sum followed by that call.
template <typename T> struct SumEpilogue {
    const T* bias = nullptr;
    FastDiv div_cols;
    int ncols = 1, relu = 0;
    __device__ __forceinline__ T apply(T s, i64 i) const {
        if (bias) {
            const uint32_t r = div_cols.div((uint32_t)i);
            s = s + bias[(uint32_t)i - r * (uint32_t)ncols];
            if (relu) s = s > T(0) ? s : T(0);
        }
        return s;
    }
};

template <typename T>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const T* __restrict__ part, T* __restrict__ out, i64 n, int splits,
                                                            const SumEpilogue<T> ep = SumEpilogue<T>()) {
    const i64 i = (i64)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    T s = T(0);
    int z = 0;
    for (; z + 8 <= splits; z += 8) {
        T v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = part[(i64)(z + u) * n + i];
#pragma unroll
        for (int u = 0; u < 8; ++u) s = s + v[u];
    }
    for (; z < splits; ++z) s = s + part[(i64)z * n + i];
    out[i] = ep.apply(s, i);
}

template <typename T, class Cfg, class AL, class BL, class EP>
int launch(fx_ctx* c, const AL& al, const BL& bl, const EP& ep, i64 M, i64 N, i64 K, int splits, int kps) {
    const i64 gx = fx::ceil_div(N, Cfg::BN), gy = fx::ceil_div(M, Cfg::BM);
    FX_REQUIRE(gx <= 0x7fffffff && gy <= 65535 && splits >= 1 && splits <= 65535, "implicit GEMM grid out of range");
    FX_REQUIRE(K >= 1, "implicit GEMM needs K >= 1");
    FX_LAUNCH(dim3((unsigned)gx, (unsigned)gy, (unsigned)splits), dim3(Cfg::NT), 0, c->stream, (
        al, bl, ep, (int)K, kps), igemm_kernel<T, Cfg, AL, BL, EP>);
    FX_LAUNCH_CHECK();
    return FX_OK;
}

template <typename T, class Cfg, class AL, class BL, class EP, int NP>
int launch_multi(fx_ctx* c, const MultiProblem<AL, BL, EP, NP>& mp, int count) {
    int gx = 0, gy = 0;
    for (int z = 0; z < count; ++z) {
        FX_REQUIRE(mp.K[z] >= 1, "implicit GEMM needs K >= 1");
        gx = std::max(gx, mp.tiles_n[z]);
        gy = std::max(gy, mp.tiles_m[z]);
    }
    FX_REQUIRE(count >= 1 && count <= NP && gx >= 1 && gy >= 1 && gy <= 65535, "implicit GEMM grid out of range");
    FX_LAUNCH(dim3((unsigned)gx, (unsigned)gy, (unsigned)count), dim3(Cfg::NT), 0, c->stream, (mp), igemm_multi_kernel<T, Cfg, AL, BL, EP, NP>);
    FX_LAUNCH_CHECK();
    return FX_OK;
}

// Same sum for few outputs and many splits: G threads share one output, thread g adds splits g, g+G, ... in
// order, then the G partial sums are added in order of g.  The grouping depends only on (n, splits), so the
// result is reproducible run to run; it differs from the single-chain order by rounding only.
template <typename T, int G>
__global__ __launch_bounds__(256) void splitk_reduce_grouped_kernel(const T* __restrict__ part, T* __restrict__ out, i64 n, int splits,
                                                                    const SumEpilogue<T> ep = SumEpilogue<T>()) {
    constexpr int COLS = 256 / G;
    __shared__ T sm[G][COLS];
    const int col = threadIdx.x % COLS, g = threadIdx.x / COLS;
    const i64 i = (i64)blockIdx.x * COLS + col;
    T s = T(0);
    if (i < n) {
        int z = g;
        for (; z + 7 * G < splits; z += 8 * G) {
            T v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = part[(i64)(z + u * G) * n + i];
#pragma unroll
            for (int u = 0; u < 8; ++u) s = s + v[u];
        }
        for (; z < splits; z += G) s = s + part[(i64)z * n + i];
    }
    sm[g][col] = s;
    __syncthreads();
    if (g == 0 && i < n) {
        T t = sm[0][col];
#pragma unroll
        for (int u = 1; u < G; ++u) t = t + sm[u][col];
        out[i] = ep.apply(t, i);
    }
}

// bias (with ncols, relu): the epilogue above; n must then fit 32 bits
template <typename T>
int launch_splitk_reduce(fx_ctx* c, const T* part, T* out, i64 n, int splits, const T* bias = nullptr, i64 ncols = 1, int relu = 0) {
    SumEpilogue<T> ep;
    if (bias) {
        FX_REQUIRE(n <= 0x7fffffff && ncols >= 1 && ncols <= 0x7fffffff, "split-K sum with bias: %lld outputs exceed 2^31", (long long)n);
        ep.bias = bias; ep.ncols = (int)ncols; ep.relu = relu; ep.div_cols = FastDiv((uint32_t)ncols);
    }
    if (splits >= 128 && n <= (1 << 16))
        FX_LAUNCH(dim3((unsigned)fx::ceil_div(n, 16)), dim3(256), 0, c->stream, (part, out, n, splits, ep), splitk_reduce_grouped_kernel<T, 16>);
    else if (splits >= 32 && n <= (1 << 18))
        FX_LAUNCH(dim3((unsigned)fx::ceil_div(n, 64)), dim3(256), 0, c->stream, (part, out, n, splits, ep), splitk_reduce_grouped_kernel<T, 4>);
    else
        FX_LAUNCH(dim3((unsigned)fx::ceil_div(n, 256)), dim3(256), 0, c->stream, (part, out, n, splits, ep), splitk_reduce_kernel<T>);
    FX_LAUNCH_CHECK();
    return FX_OK;
}

// Partial sums that carry a second, short result behind the first ([n1] then [n2] floats per split, `stride` apart): both are
// added over the splits and go to their own tensors.  G threads share an output (thread g adds partials g, g + G, ... in order,
// then the G sums are added in order of g; G = 1: one chain): the orders of splitk_reduce_kernel / splitk_reduce_grouped_kernel,
// chosen by the same rule, so the first result has the bits launch_splitk_reduce gives it.
template <typename T, int G>
__global__ __launch_bounds__(256) void splitk_reduce_pair_kernel(const T* __restrict__ part, i64 stride, int splits, T* __restrict__ out1,
                                                                 i64 n1, T* __restrict__ out2, i64 n2) {
    constexpr int COLS = 256 / G;
    __shared__ T sm[G][COLS];
    const int col = threadIdx.x % COLS, g = threadIdx.x / COLS;
    const i64 i = (i64)blockIdx.x * COLS + col;
    T s = T(0);
    if (i < n1 + n2) {
        int z = g;
        for (; z + 7 * G < splits; z += 8 * G) {
            T v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = part[(i64)(z + u * G) * stride + i];
#pragma unroll
            for (int u = 0; u < 8; ++u) s = s + v[u];
        }
        for (; z < splits; z += G) s = s + part[(i64)z * stride + i];
    }
    if (G > 1) {
        sm[g][col] = s;
        __syncthreads();
    }
    if (g == 0 && i < n1 + n2) {
        T t = s;
        if (G > 1) {
            t = sm[0][col];
#pragma unroll
            for (int u = 1; u < G; ++u) t = t + sm[u][col];
        }
        if (i < n1) out1[i] = t;
        else out2[i - n1] = t;
    }
}
template <typename T>
int launch_splitk_reduce_pair(fx_ctx* c, const T* part, i64 stride, int splits, T* out1, i64 n1, T* out2, i64 n2) {
    const i64 n = n1 + n2;
    FX_REQUIRE(stride >= n && n <= 0x7fffffffll, "split-K pair sum: bad sizes");
    if (splits >= 128 && n1 <= (1 << 16))
        FX_LAUNCH(dim3((unsigned)fx::ceil_div(n, (i64)16)), dim3(256), 0, c->stream, (part, stride, splits, out1, n1, out2, n2), splitk_reduce_pair_kernel<T, 16>);
    else if (splits >= 32 && n1 <= (1 << 18))
        FX_LAUNCH(dim3((unsigned)fx::ceil_div(n, (i64)64)), dim3(256), 0, c->stream, (part, stride, splits, out1, n1, out2, n2), splitk_reduce_pair_kernel<T, 4>);
    else
        FX_LAUNCH(dim3((unsigned)fx::ceil_div(n, (i64)256)), dim3(256), 0, c->stream, (part, stride, splits, out1, n1, out2, n2), splitk_reduce_pair_kernel<T, 1>);
    FX_LAUNCH_CHECK();
    return FX_OK;
}

template <typename T>
__global__ __launch_bounds__(256) void zero_kernel(T* __restrict__ out, i64 n) {
    const i64 i = (i64)blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = T(0);
}
template <typename T>
int launch_zero(fx_ctx* c, T* out, i64 n) {
    if (n == 0) return FX_OK;
    FX_LAUNCH(dim3((unsigned)fx::ceil_div(n, 256)), dim3(256), 0, c->stream, (out, n), zero_kernel<T>);
    FX_LAUNCH_CHECK();
    return FX_OK;
}

// Picks the number of K splits so that about `want_blocks` blocks exist; returns kps (multiple of BK).
inline int choose_splits(i64 tiles, i64 K, int BK, i64 want_blocks, int* kps_out) {
    i64 splits = 1;
    if (tiles < want_blocks) splits = std::min<i64>(fx::ceil_div(want_blocks, tiles), std::max<i64>(1, K / (4 * BK)));
    i64 kps = fx::ceil_div(fx::ceil_div(K, splits), BK) * BK;
    splits = fx::ceil_div(K, kps);
    *kps_out = (int)kps;
    return (int)splits;
}

inline ConvShape make_shape(i64 B, i64 Cin, i64 H, i64 W, i64 Cout, i64 kh, i64 kw, i64 sh, i64 sw, i64 ph, i64 pw) {
    ConvShape s;
    s.B = (int)B; s.Cin = (int)Cin; s.H = (int)H; s.W = (int)W; s.Cout = (int)Cout;
    s.kh = (int)kh; s.kw = (int)kw; s.sh = (int)sh; s.sw = (int)sw; s.ph = (int)ph; s.pw = (int)pw;
    s.oh = (int)((H + 2 * ph - kh) / sh + 1);
    s.ow = (int)((W + 2 * pw - kw) / sw + 1);
    s.div_L = FastDiv((uint32_t)(s.oh * s.ow));
    s.div_ow = FastDiv((uint32_t)s.ow);
    s.div_KK = FastDiv((uint32_t)(kh * kw));
    s.div_kw = FastDiv((uint32_t)kw);
    s.div_HW = FastDiv((uint32_t)(H * W));
    s.div_W = FastDiv((uint32_t)W);
    s.div_sh = FastDiv((uint32_t)sh);
    s.div_sw = FastDiv((uint32_t)sw);
    s.div_Cin = FastDiv((uint32_t)Cin);
    s.div_Cout = FastDiv((uint32_t)Cout);
    return s;
}

}  // namespace igemm
