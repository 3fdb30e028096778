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
// Global loads for slab i+1 are issued before the MFMA loop of slab i, so their latency hides behind the matrix
// pipe; two or more blocks are resident per CU so one block's barriers overlap another block's MFMAs.
// Index arithmetic uses 32-bit tile coordinates (hosts check M, N, K < 2^31) and 64-bit addresses.
#pragma once
#include <climits>
#include <algorithm>

#include "common.hpp"

namespace igemm {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef double f64x4 __attribute__((ext_vector_type(4)));

// Division by a runtime constant as multiply-high + shift (exact for all 32-bit n).
struct FastDiv {
    uint32_t d, m, s;
    FastDiv() : d(1), m(1), s(0) {}
    explicit FastDiv(uint32_t d_) : d(d_) {
        s = 0;
        while ((1ull << s) < d) ++s;
        m = (uint32_t)((((1ull << 32) * ((1ull << s) - d)) / d) + 1);
    }
    __device__ __forceinline__ uint32_t div(uint32_t n) const { return (uint32_t)(((uint64_t)__umulhi(n, m) + n) >> s); }
};

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
    static constexpr int LD = KMAJOR ? BMN + 1 : BMN;  // LDS row pitch; +1 spreads the transposing writes over banks
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
        const T* p; i64 ld; int MN, origin, tid;
        __device__ __forceinline__ Dev(const MatLoader& L, int origin_, int tid_) : p(L.p), ld(L.ld), MN(L.MN), origin(origin_), tid(tid_) {}
        __device__ __forceinline__ void load(int k0, int kend, T (&r)[Map::CNT]) const {
            if (KMAJOR_) {
                const int k = k0 + tid % BK;
                const bool kok = k < kend;
#pragma unroll
                for (int i = 0; i < Map::CNT; ++i) {
                    const int mn = origin + Map::mn_of(tid, i);
                    r[i] = (kok && mn < MN) ? p[(i64)mn * ld + k] : T(0);
                }
            } else {
                const int mn = origin + tid % BMN;
                const bool ok = mn < MN;
                const int krow = __builtin_amdgcn_readfirstlane(tid / BMN);
#pragma unroll
                for (int i = 0; i < Map::CNT; ++i) {
                    const int k = k0 + krow + i * Map::STEP;
                    r[i] = (ok && k < kend) ? p[(i64)k * ld + mn] : T(0);
                }
            }
        }
    };
};

// ---- convolution geometry shared by the conv loaders -------------------------------------------------------
struct ConvShape {
    int B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, oh, ow;
    FastDiv div_L, div_ow, div_KK, div_kw, div_HW, div_W, div_sh, div_sw;
};

// Forward B operand: B(k = (c,ky,kx), n = (b,oy,ox)) = x[b, c, oy*sh + ky - ph, ox*sw + kx - pw] (0 outside).
// Contiguous along n.  The pixel of a thread is fixed for the whole kernel; k is wave-uniform.
template <typename T> struct ConvFwdB {
    static constexpr bool KMAJOR = false;
    const T* x;
    ConvShape s;
    int N;
    template <int BMN, int BK, int NT> struct Dev {
        typedef SlabMap<BMN, BK, NT, false> Map;
        const T* base; const ConvShape& s; int iy0, ix0, krow; bool ok;
        __device__ __forceinline__ Dev(const ConvFwdB& L, int origin, int tid) : s(L.s) {
            const int n = origin + tid % BMN;
            ok = n < L.N;
            const uint32_t nn = ok ? n : 0;
            const uint32_t b = s.div_L.div(nn), l = nn - b * (s.oh * s.ow);
            const uint32_t oy = s.div_ow.div(l), ox = l - oy * s.ow;
            base = L.x + (i64)b * s.Cin * s.H * s.W;
            iy0 = (int)oy * s.sh - s.ph;
            ix0 = (int)ox * s.sw - s.pw;
            krow = __builtin_amdgcn_readfirstlane(tid / BMN);
        }
        __device__ __forceinline__ void load(int k0, int kend, T (&r)[Map::CNT]) const {
            const int KK = s.kh * s.kw;
#pragma unroll
            for (int i = 0; i < Map::CNT; ++i) {
                const int k = k0 + krow + i * Map::STEP;
                const uint32_t c = s.div_KK.div(k), rr = k - c * KK;
                const uint32_t ky = s.div_kw.div(rr), kx = rr - ky * s.kw;
                const int iy = iy0 + (int)ky, ix = ix0 + (int)kx;
                const bool in = ok && k < kend && (unsigned)iy < (unsigned)s.H && (unsigned)ix < (unsigned)s.W;
                r[i] = in ? base[((int)c * s.H + iy) * s.W + ix] : T(0);
            }
        }
    };
};

// Data-gradient B operand: B(k = (oc,ky,kx), n = (b,y,x)) = g[b, oc, (y+ph-ky)/sh, (x+pw-kx)/sw] when both
// quotients are exact and inside the output plane, else 0.  This is the gather form of col2im: every input pixel
// is owned by exactly one accumulator, so there are no races and no atomics.
template <typename T> struct ConvDgradB {
    static constexpr bool KMAJOR = false;
    const T* g;
    ConvShape s;
    int N;  // B*H*W
    template <int BMN, int BK, int NT> struct Dev {
        typedef SlabMap<BMN, BK, NT, false> Map;
        const T* base; const ConvShape& s; int yp, xp, krow; bool ok;
        __device__ __forceinline__ Dev(const ConvDgradB& L, int origin, int tid) : s(L.s) {
            const int n = origin + tid % BMN;
            ok = n < L.N;
            const uint32_t nn = ok ? n : 0;
            const uint32_t b = s.div_HW.div(nn), p = nn - b * (s.H * s.W);
            const uint32_t y = s.div_W.div(p), x = p - y * s.W;
            base = L.g + (i64)b * s.Cout * s.oh * s.ow;
            yp = (int)y + s.ph;
            xp = (int)x + s.pw;
            krow = __builtin_amdgcn_readfirstlane(tid / BMN);
        }
        __device__ __forceinline__ void load(int k0, int kend, T (&r)[Map::CNT]) const {
            const int KK = s.kh * s.kw;
            const bool unit = (s.sh == 1 && s.sw == 1);
#pragma unroll
            for (int i = 0; i < Map::CNT; ++i) {
                const int k = k0 + krow + i * Map::STEP;
                const uint32_t oc = s.div_KK.div(k), rr = k - oc * KK;
                const uint32_t ky = s.div_kw.div(rr), kx = rr - ky * s.kw;
                const int ty = yp - (int)ky, tx = xp - (int)kx;
                bool in = ok && k < kend && ty >= 0 && tx >= 0;
                int cy = ty, cx = tx;
                if (!unit) {
                    const uint32_t uy = in ? (uint32_t)ty : 0u, ux = in ? (uint32_t)tx : 0u;
                    cy = (int)s.div_sh.div(uy);
                    cx = (int)s.div_sw.div(ux);
                    in = in && (cy * s.sh == ty) && (cx * s.sw == tx);
                }
                in = in && cy < s.oh && cx < s.ow;
                r[i] = in ? base[((int)oc * s.oh + cy) * s.ow + cx] : T(0);
            }
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
        const T* g; const ConvShape& s; int origin, tid;
        __device__ __forceinline__ Dev(const ConvWgradA& L, int origin_, int tid_) : g(L.g), s(L.s), origin(origin_), tid(tid_) {}
        __device__ __forceinline__ void load(int k0, int kend, T (&r)[Map::CNT]) const {
            const int k = k0 + tid % BK;
            const bool kok = k < kend;
            const int L = s.oh * s.ow;
            const uint32_t kk = kok ? k : 0;
            const uint32_t b = s.div_L.div(kk), l = kk - b * L;
            const T* p = g + (i64)b * s.Cout * L + l;
#pragma unroll
            for (int i = 0; i < Map::CNT; ++i) {
                const int m = origin + Map::mn_of(tid, i);
                r[i] = (kok && m < s.Cout) ? p[(i64)m * L] : T(0);
            }
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
        const T* x; const ConvShape& s; int tid;
        int off[Map::CNT];   // c*H*W + (ky-ph)*W + (kx-pw)
        int kyx[Map::CNT];   // (ky-ph) << 16 | ((kx-pw) & 0xffff); INT_MIN when the column is out of range
        __device__ __forceinline__ Dev(const ConvWgradB& L, int origin, int tid_) : x(L.x), s(L.s), tid(tid_) {
            const int KK = s.kh * s.kw;
#pragma unroll
            for (int i = 0; i < Map::CNT; ++i) {
                const int n = origin + Map::mn_of(tid, i);
                if (n < L.N) {
                    const uint32_t c = s.div_KK.div(n), rr = n - c * KK;
                    const uint32_t ky = s.div_kw.div(rr), kx = rr - ky * s.kw;
                    const int dy = (int)ky - s.ph, dx = (int)kx - s.pw;
                    off[i] = ((int)c * s.H + dy) * s.W + dx;
                    kyx[i] = (dy << 16) | (dx & 0xffff);
                } else {
                    off[i] = 0;
                    kyx[i] = INT_MIN;
                }
            }
        }
        __device__ __forceinline__ void load(int k0, int kend, T (&r)[Map::CNT]) const {
            const int k = k0 + tid % BK;
            const bool kok = k < kend;
            const uint32_t kk = kok ? k : 0;
            const int L = s.oh * s.ow;
            const uint32_t b = s.div_L.div(kk), l = kk - b * L;
            const uint32_t oy = s.div_ow.div(l), ox = l - oy * s.ow;
            const int y0 = (int)oy * s.sh, x0 = (int)ox * s.sw;
            const T* p = x + (i64)b * s.Cin * s.H * s.W + y0 * s.W + x0;
#pragma unroll
            for (int i = 0; i < Map::CNT; ++i) {
                const int dy = kyx[i] >> 16, dx = (int)(short)(kyx[i] & 0xffff);
                const bool in = kok && kyx[i] != INT_MIN && (unsigned)(y0 + dy) < (unsigned)s.H && (unsigned)(x0 + dx) < (unsigned)s.W;
                r[i] = in ? p[off[i]] : T(0);
            }
        }
    };
};

// ---- epilogues ---------------------------------------------------------------------------------------------
// Row-major matrix (also used for split-K partials: split z goes to p + z*split_stride).
template <typename T> struct MatStore {
    T* p;
    i64 ld, split_stride;
    int M, N;
    struct Col { T* q; };
    __device__ __forceinline__ Col col(int n, int split) const { return Col{n < N ? p + (i64)split * split_stride + n : nullptr}; }
    __device__ __forceinline__ void put(const Col& c, int m, T v) const { if (c.q && m < M) c.q[(i64)m * ld] = v; }
};
// NCHW tensor: row m = channel, column n = (b, l) -> p[(b*C + m)*L + l].
template <typename T> struct NchwStore {
    T* p;
    int C, L, N;
    FastDiv div_L;
    struct Col { T* q; };
    __device__ __forceinline__ Col col(int n, int) const {
        if (n >= N) return Col{nullptr};
        const uint32_t b = div_L.div(n), l = n - b * L;
        return Col{p + (i64)b * C * L + l};
    }
    __device__ __forceinline__ void put(const Col& c, int m, T v) const { if (c.q && m < C) c.q[(i64)m * L] = v; }
};

// ---- the kernel -------------------------------------------------------------------------------------------
// grid (N tiles, M tiles, K splits).  Split z covers k in [z*kps, min(K, (z+1)*kps)), kps a multiple of BK.
template <typename T, class Cfg, class AL, class BL, class EP>
__global__ __launch_bounds__(Cfg::NT) void igemm_kernel(AL al, BL bl, EP ep, int K, int kps) {
    typedef Mfma<T> MF;
    constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, NT = Cfg::NT;
    constexpr int TM = Cfg::WM / MF::BLK, TN = Cfg::WN / MF::BLK;
    static_assert(Cfg::WM % MF::BLK == 0 && Cfg::WN % MF::BLK == 0 && BK % MF::KSTEP == 0, "tile must be a multiple of the MFMA block");
    typedef typename AL::template Dev<BM, BK, NT> ADev;
    typedef typename BL::template Dev<BN, BK, NT> BDev;
    typedef typename ADev::Map AMap;
    typedef typename BDev::Map BMap;

    __shared__ T As[BK * AMap::LD];
    __shared__ T Bs[BK * BMap::LD];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int bm = blockIdx.y * BM, bn = blockIdx.x * BN, split = blockIdx.z;
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

    const int lrow = lane / MF::BLK, lcol = lane % MF::BLK;
    for (int k0 = kbeg; k0 < kend; k0 += BK) {
        __syncthreads();  // everyone is done reading the previous slab
        AMap::store(As, ra, tid);
        BMap::store(Bs, rb, tid);
        __syncthreads();
        if (k0 + BK < kend) {  // prefetch the next slab; latency hides behind the MFMA loop below
            ad.load(k0 + BK, kend, ra);
            bd.load(k0 + BK, kend, rb);
        }
#pragma unroll
        for (int kk = 0; kk < BK; kk += MF::KSTEP) {
            T a[TM], b[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) a[i] = As[(kk + lrow) * AMap::LD + wm0 + i * MF::BLK + lcol];
#pragma unroll
            for (int j = 0; j < TN; ++j) b[j] = Bs[(kk + lrow) * BMap::LD + wn0 + j * MF::BLK + lcol];
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[i][j] = MF::mma(a[i], b[j], acc[i][j]);
        }
    }

#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int n = bn + wn0 + j * MF::BLK + lcol;
        const typename EP::Col cc = ep.col(n, split);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int e = 0; e < MF::NACC; ++e) ep.put(cc, bm + wm0 + i * MF::BLK + MF::row(e, lane), acc[i][j][e]);
    }
}

// Sums split-K partials in split order (deterministic) into the final buffer.
template <typename T>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const T* __restrict__ part, T* __restrict__ out, i64 n, int splits) {
    const i64 i = (i64)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    T s = part[i];
    for (int z = 1; z < splits; ++z) s = s + part[(i64)z * n + i];
    out[i] = s;
}

template <typename T, class Cfg, class AL, class BL, class EP>
int launch(fx_ctx* c, const AL& al, const BL& bl, const EP& ep, i64 M, i64 N, i64 K, int splits, int kps) {
    const i64 gx = fx::ceil_div(N, Cfg::BN), gy = fx::ceil_div(M, Cfg::BM);
    FX_REQUIRE(gx <= 0x7fffffff && gy <= 65535 && splits >= 1 && splits <= 65535, "implicit GEMM grid out of range");
    igemm_kernel<T, Cfg, AL, BL, EP><<<dim3((unsigned)gx, (unsigned)gy, (unsigned)splits), dim3(Cfg::NT), 0, c->stream>>>(
        al, bl, ep, (int)K, kps);
    FX_LAUNCH_CHECK();
    return FX_OK;
}

template <typename T>
int launch_splitk_reduce(fx_ctx* c, const T* part, T* out, i64 n, int splits) {
    splitk_reduce_kernel<T><<<dim3((unsigned)fx::ceil_div(n, 256)), dim3(256), 0, c->stream>>>(part, out, n, splits);
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
    zero_kernel<T><<<dim3((unsigned)fx::ceil_div(n, 256)), dim3(256), 0, c->stream>>>(out, n);
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
    return s;
}

}  // namespace igemm
