// Axis reductions (sum / mean / max with first-occurrence argmax) and the axis softmax.
// Replaces kernels/reduction.cu and softmax_batch_axis of kernels/activations.cu.  The reference launches one
// 32-lane-shuffle block per output element and walks the axis with stride `inner` (uncoalesced when inner > 1);
// here every access is a coalesced 16-byte vector and the work is split so that thousands of wave64 blocks are in
// flight, because these kernels are HBM-bound: sizeof(T) * (outer*axis*inner + outer*inner) bytes per call.
//
// Two shapes of the contiguous [outer, axis, inner] view:
//   inner == 1 : "row" reduction.  grid (S, outer): block (s, o) reduces slice s of row o.
//   inner  > 1 : "column" reduction.  A wave covers 64 vectors of adjacent columns; the four waves of a block
//                take interleaved rows of the axis slice; grid (column tiles, S, outer).
// When the axis is split (S > 1) the per-slice partials go to library scratch and a second small kernel combines
// them in slice order; no atomics, so results are deterministic run to run.
// Max takes strictly greater values starting from the lowest finite T (src/backend/storage/cpu.rs:1231-1234);
// the recorded index is the first position along the axis that attains the maximum.
#include <cstdlib>
#include <limits>

#include "common.hpp"

namespace {

constexpr i64 NO_INDEX = INT64_MAX;
// Inputs that cannot stay in the 256 MiB Infinity Cache between their producer and this read -- three quarters of its size and
// more -- are read with cache-bypassing loads.  Measured on 8192^2 f32 (256 MiB) with three inputs in rotation, so that every
// read comes from HBM: sum over all 51.4 -> 45.1 us, axis 0 47.6 -> 46.2, axis 1 44.0 -> 40.8, max over all 53.4 -> 47.2 us; the
// same tensor re-read in place (the cache's best case) loses 3 us (41.6 -> 44.6 us).
// (Adding the slice partials in the same launch -- the block that draws a row's last ticket after a device-scope fence adds
// them -- was measured at 69.8 against 44.7 us for the sum over all: 763 release fences cost far more than the second launch.)
constexpr i64 STREAM_BYTES = 192ll << 20;

template <typename T> struct Vec16;
template <> struct Vec16<float> { typedef float4 type; static constexpr int N = 4; };
template <> struct Vec16<double> { typedef double2 type; static constexpr int N = 2; };
template <typename T> __device__ __forceinline__ T vget(const typename Vec16<T>::type& v, int i);
template <> __device__ __forceinline__ float vget<float>(const float4& v, int i) { return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w; }
template <> __device__ __forceinline__ double vget<double>(const double2& v, int i) { return i == 0 ? v.x : v.y; }

// 16-byte load that bypasses the caches when STREAM is set (inputs much larger than L2 are read exactly once)
typedef float nt_f4 __attribute__((ext_vector_type(4)));
typedef double nt_d2 __attribute__((ext_vector_type(2)));
template <bool STREAM> __device__ __forceinline__ float4 ld16(const float4* p) {
    if (!STREAM) return *p;
    const nt_f4 v = __builtin_nontemporal_load(reinterpret_cast<const nt_f4*>(p));
    return float4{v.x, v.y, v.z, v.w};
}
template <bool STREAM> __device__ __forceinline__ double2 ld16(const double2* p) {
    if (!STREAM) return *p;
    const nt_d2 v = __builtin_nontemporal_load(reinterpret_cast<const nt_d2*>(p));
    return double2{v.x, v.y};
}

template <typename T> __device__ __forceinline__ T lowest();
template <> __device__ __forceinline__ float lowest<float>() { return -3.402823466e+38f; }
template <> __device__ __forceinline__ double lowest<double>() { return -1.7976931348623157e+308; }

__device__ __forceinline__ i64 shfl_down_i64(i64 v, int d) {
    int lo = (int)(v & 0xffffffffll), hi = (int)(v >> 32);
    lo = __shfl_down(lo, d, 64);
    hi = __shfl_down(hi, d, 64);
    return ((i64)hi << 32) | (unsigned int)lo;
}
__device__ __forceinline__ double shfl_down_t(double v, int d) { return __shfl_down(v, d, 64); }
__device__ __forceinline__ float shfl_down_t(float v, int d) { return __shfl_down(v, d, 64); }

// Accumulator: value (+ index for the extrema).  IS_MAX: 0 = sum (ignores idx), 1 = maximum, 2 = minimum,
// 3 = product (ignores idx; kernels/reduction.cu:232-301 starts from 1 and multiplies), 4 / 5 = maximum / minimum whose
// position nobody asked for: the same comparisons on the values, without the 64-bit index that rides along in 1 / 2
// (three more selects and a 64-bit add per element: 46.8 against 44.9 us over 2^26 floats).
#define EXTREMUM(M) ((M) == 1 || (M) == 2)
// The extrema start from the lowest / highest finite T and take strictly greater / smaller values
// (cpu.rs:1231-1234, 1240-1252), so the first position attaining the extremum wins.
template <typename T, int IS_MAX> struct Acc {
    T v;
    i64 i;
    __device__ __forceinline__ void init() {
        v = (IS_MAX == 1 || IS_MAX == 4) ? lowest<T>() : (IS_MAX == 2 || IS_MAX == 5) ? -lowest<T>() : IS_MAX == 3 ? T(1) : T(0);
        i = NO_INDEX;
    }
    // element x at axis position p, visited in increasing p by this thread
    __device__ __forceinline__ void take(T x, i64 p) {
        if (IS_MAX == 1) { if (x > v) { v = x; i = p; } }
        else if (IS_MAX == 2) { if (x < v) { v = x; i = p; } }
        else if (IS_MAX == 3) v = v * x;
        else if (IS_MAX == 4) { if (x > v) v = x; }
        else if (IS_MAX == 5) { if (x < v) v = x; }
        else v = v + x;
    }
    // merge another accumulator (any order): ties go to the smaller index
    __device__ __forceinline__ void merge(T ov, i64 oi) {
        if (IS_MAX == 1) { if (ov > v || (ov == v && oi < i)) { v = ov; i = oi; } }
        else if (IS_MAX == 2) { if (ov < v || (ov == v && oi < i)) { v = ov; i = oi; } }
        else if (IS_MAX == 3) v = v * ov;
        else if (IS_MAX == 4) { if (ov > v) v = ov; }
        else if (IS_MAX == 5) { if (ov < v) v = ov; }
        else v = v + ov;
    }
};

template <typename T, int IS_MAX>
__device__ __forceinline__ void wave_reduce(Acc<T, IS_MAX>& a) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        const T ov = shfl_down_t(a.v, d);
        i64 oi = NO_INDEX;
        if (EXTREMUM(IS_MAX)) oi = shfl_down_i64(a.i, d);
        a.merge(ov, oi);
    }
}

// ---- row reduction (inner == 1) ---------------------------------------------------------------------------
// grid (S, outer), 256 threads.  Slice s covers [s*chunk, min(axis, (s+1)*chunk)).  VEC: 16-byte loads (requires
// axis % N == 0, chunk % N == 0 and a 16-byte aligned base).  Output slot o*S + s.
template <typename T, int IS_MAX, bool VEC, bool STREAM>
__global__ __launch_bounds__(256) void row_reduce_kernel(const T* __restrict__ in, T* __restrict__ out, i64* __restrict__ idx_out,
                                                         i64 axis, i64 chunk, T scale) {
    constexpr int N = Vec16<T>::N;
    typedef typename Vec16<T>::type V;
    const i64 o = blockIdx.y, s = blockIdx.x, S = gridDim.x;
    const i64 beg = s * chunk, end = min(axis, beg + chunk);
    const T* row = in + o * axis;
    Acc<T, IS_MAX> acc;
    acc.init();
    if (VEC) {
        const V* rv = reinterpret_cast<const V*>(row);
        const i64 vbeg = beg / N, vend = end / N;
        i64 p = vbeg + threadIdx.x;
        if constexpr (IS_MAX == 1 || IS_MAX == 2 || IS_MAX == 4 || IS_MAX == 5) {
            // An extremum is a chain of dependent compare + select pairs, and a long slice runs with few waves per SIMD to hide
            // it behind: one accumulator per vector in flight, merged afterwards (each visits its elements in increasing
            // position and a merge gives ties to the smaller one, so the first position attaining the extremum still wins).
            Acc<T, IS_MAX> a1, a2, a3;
            a1.init(); a2.init(); a3.init();
            for (; p + 3 * 256 < vend; p += 4 * 256) {
                V r0 = ld16<STREAM>(rv + p), r1 = ld16<STREAM>(rv + p + 256), r2 = ld16<STREAM>(rv + p + 512), r3 = ld16<STREAM>(rv + p + 768);
#pragma unroll
                for (int e = 0; e < N; ++e) {
                    acc.take(vget<T>(r0, e), p * N + e);
                    a1.take(vget<T>(r1, e), (p + 256) * N + e);
                    a2.take(vget<T>(r2, e), (p + 512) * N + e);
                    a3.take(vget<T>(r3, e), (p + 768) * N + e);
                }
            }
            acc.merge(a1.v, a1.i);
            acc.merge(a2.v, a2.i);
            acc.merge(a3.v, a3.i);
        } else
        for (; p + 3 * 256 < vend; p += 4 * 256) {
            V r0 = ld16<STREAM>(rv + p), r1 = ld16<STREAM>(rv + p + 256), r2 = ld16<STREAM>(rv + p + 512), r3 = ld16<STREAM>(rv + p + 768);
#pragma unroll
            for (int e = 0; e < N; ++e) acc.take(vget<T>(r0, e), p * N + e);
#pragma unroll
            for (int e = 0; e < N; ++e) acc.take(vget<T>(r1, e), (p + 256) * N + e);
#pragma unroll
            for (int e = 0; e < N; ++e) acc.take(vget<T>(r2, e), (p + 512) * N + e);
#pragma unroll
            for (int e = 0; e < N; ++e) acc.take(vget<T>(r3, e), (p + 768) * N + e);
        }
        for (; p < vend; p += 256) {
            V r0 = ld16<STREAM>(rv + p);
#pragma unroll
            for (int e = 0; e < N; ++e) acc.take(vget<T>(r0, e), p * N + e);
        }
    } else {
        for (i64 p = beg + threadIdx.x; p < end; p += 256) acc.take(row[p], p);
    }
    wave_reduce(acc);
    __shared__ T sv[4];
    __shared__ i64 si[4];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0) { sv[wave] = acc.v; si[wave] = acc.i; }
    __syncthreads();
    if (threadIdx.x == 0) {
        Acc<T, IS_MAX> r;
        r.v = sv[0]; r.i = si[0];
        for (int w = 1; w < 4; ++w) r.merge(sv[w], si[w]);
        const i64 slot = o * S + s;
        out[slot] = EXTREMUM(IS_MAX) ? r.v : r.v * scale;
        if (EXTREMUM(IS_MAX) && idx_out) idx_out[slot] = (S == 1 && r.i == NO_INDEX) ? 0 : r.i;
    }
}

// Short rows: G = power of two >= axis lanes per row (G <= 64), 64/G rows per wave, 4 waves per block.
template <typename T, int IS_MAX>
__global__ __launch_bounds__(256) void short_row_reduce_kernel(const T* __restrict__ in, T* __restrict__ out,
                                                               i64* __restrict__ idx_out, i64 outer, i64 axis, int G, T scale) {
    const int lane = threadIdx.x & 63;
    const i64 rows_per_block = (256 / G);
    const i64 o = (i64)blockIdx.x * rows_per_block + threadIdx.x / G;
    const int a = threadIdx.x % G;
    Acc<T, IS_MAX> acc;
    acc.init();
    if (o < outer && a < axis) acc.take(in[o * axis + a], a);
    for (int d = G >> 1; d >= 1; d >>= 1) {
        const T ov = shfl_down_t(acc.v, d);
        i64 oi = NO_INDEX;
        if (EXTREMUM(IS_MAX)) oi = shfl_down_i64(acc.i, d);
        if ((lane % G) + d < G) acc.merge(ov, oi);
    }
    if (a == 0 && o < outer) {
        out[o] = EXTREMUM(IS_MAX) ? acc.v : acc.v * scale;
        if (EXTREMUM(IS_MAX) && idx_out) idx_out[o] = acc.i == NO_INDEX ? 0 : acc.i;
    }
}

// Short rows whose length is a multiple of the 16-byte vector (rows of up to 64 vectors): a lane takes one vector of a row, GV =
// power of two >= vectors per row lanes share a row, and a thread keeps the vectors of U rows in flight (a block reads U
// contiguous stretches of 4 KiB when the row length is a power of two).  One element per lane, as above, left a [256,32,32,32]
// sum over the last axis at 24 us for 33.5 MB.
template <typename T, int IS_MAX>
__global__ __launch_bounds__(256) void short_row_vec_kernel(const T* __restrict__ in, T* __restrict__ out, i64* __restrict__ idx_out,
                                                            i64 outer, int axis_v, int GV, T scale) {
    constexpr int N = Vec16<T>::N, U = 4;
    typedef typename Vec16<T>::type V;
    const int lane = threadIdx.x & 63;
    const int a = threadIdx.x % GV;
    const i64 rows_per_pass = 256 / GV;
    const i64 row0 = (i64)blockIdx.x * U * rows_per_pass + threadIdx.x / GV;
    V v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const i64 o = row0 + u * rows_per_pass;
        if (o < outer && a < axis_v) v[u] = ld16<false>(reinterpret_cast<const V*>(in + o * axis_v * N) + a);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const i64 o = row0 + u * rows_per_pass;
        Acc<T, IS_MAX> acc;
        acc.init();
        if (o < outer && a < axis_v) {
#pragma unroll
            for (int e = 0; e < N; ++e) acc.take(vget<T>(v[u], e), a * N + e);
        }
        for (int d = GV >> 1; d >= 1; d >>= 1) {
            const T ov = shfl_down_t(acc.v, d);
            i64 oi = NO_INDEX;
            if (EXTREMUM(IS_MAX)) oi = shfl_down_i64(acc.i, d);
            if ((lane % GV) + d < GV) acc.merge(ov, oi);
        }
        if (a == 0 && o < outer) {
            out[o] = EXTREMUM(IS_MAX) ? acc.v : acc.v * scale;
            if (EXTREMUM(IS_MAX) && idx_out) idx_out[o] = acc.i == NO_INDEX ? 0 : acc.i;
        }
    }
}

// Combine S slice partials per output: one 256-thread block per output element, slices merged with the tie rule.
template <typename T, int IS_MAX>
__global__ __launch_bounds__(256) void combine_rows_kernel(const T* __restrict__ pv, const i64* __restrict__ pi, T* __restrict__ out,
                                                           i64* __restrict__ idx_out, i64 n_out, i64 S, T scale) {
    const i64 o = blockIdx.x;
    Acc<T, IS_MAX> acc;
    acc.init();
    for (i64 s = threadIdx.x; s < S; s += 256) acc.merge(pv[o * S + s], EXTREMUM(IS_MAX) && pi ? pi[o * S + s] : NO_INDEX);
    wave_reduce(acc);
    __shared__ T sv[4];
    __shared__ i64 si[4];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0) { sv[wave] = acc.v; si[wave] = acc.i; }
    __syncthreads();
    if (threadIdx.x == 0) {
        Acc<T, IS_MAX> r;
        r.v = sv[0]; r.i = si[0];
        for (int w = 1; w < 4; ++w) r.merge(sv[w], si[w]);
        out[o] = EXTREMUM(IS_MAX) ? r.v : r.v * scale;
        if (EXTREMUM(IS_MAX) && idx_out) idx_out[o] = r.i == NO_INDEX ? 0 : r.i;
    }
}

// ---- column reduction (inner > 1) -------------------------------------------------------------------------
// grid (col tiles, S, outer), 256 threads = 4 waves arranged as CW waves side by side x (4/CW) waves over rows.
// A wave covers 64*NV adjacent columns (NV = N when VEC else 1), so a block reads CW*64*NV contiguous elements of
// each row it visits (4 KiB at CW = 4 with 16-byte vectors); waves sharing columns take interleaved axis positions
// and are merged through LDS.  Output slot ((o*S + s) * inner + col).
// FROM_PARTIAL: the input is a partial array whose index values come from `pidx` instead of the axis position.
template <typename T, int IS_MAX, bool VEC, bool FROM_PARTIAL, int CW, bool STREAM>
__global__ __launch_bounds__(256) void col_reduce_kernel(const T* __restrict__ in, const i64* __restrict__ pidx, T* __restrict__ out,
                                                         i64* __restrict__ idx_out, i64 axis, i64 inner, i64 chunk, T scale,
                                                         int final_pass) {
    constexpr int N = VEC ? Vec16<T>::N : 1;
    constexpr int RW = 4 / CW;
    typedef typename Vec16<T>::type V;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int wc = wave % CW, wr = wave / CW;
    const i64 col = (((i64)blockIdx.x * CW + wc) * 64 + lane) * N;
    const i64 s = blockIdx.y, S = gridDim.y, o = blockIdx.z;
    const i64 beg = s * chunk, end = min(axis, beg + chunk);
    Acc<T, IS_MAX> acc[N];
#pragma unroll
    for (int e = 0; e < N; ++e) acc[e].init();
    if (col < inner) {
        const T* base = in + (o * axis) * inner + col;
        const i64* ibase = FROM_PARTIAL && EXTREMUM(IS_MAX) ? pidx + (o * axis) * inner + col : nullptr;
        i64 a = beg + wr;
        if (VEC && !FROM_PARTIAL) {
            for (; a + 7 * RW < end; a += 8 * RW) {
                V r[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) r[u] = ld16<STREAM>(reinterpret_cast<const V*>(base + (a + u * RW) * inner));
#pragma unroll
                for (int u = 0; u < 8; ++u)
#pragma unroll
                    for (int e = 0; e < N; ++e) acc[e].take(vget<T>(r[u], e), a + u * RW);
            }
            for (; a < end; a += RW) {
                V r0 = ld16<STREAM>(reinterpret_cast<const V*>(base + a * inner));
#pragma unroll
                for (int e = 0; e < N; ++e) acc[e].take(vget<T>(r0, e), a);
            }
        } else {
            for (; a < end; a += RW) {
#pragma unroll
                for (int e = 0; e < N; ++e) {
                    const T x = base[a * inner + e];
                    if (FROM_PARTIAL) acc[e].merge(x, EXTREMUM(IS_MAX) ? ibase[a * inner + e] : NO_INDEX);
                    else acc[e].take(x, a);
                }
            }
        }
    }
    __shared__ T sv[RW][CW * 64 * N];
    __shared__ i64 si[EXTREMUM(IS_MAX) ? RW : 1][EXTREMUM(IS_MAX) ? CW * 64 * N : 1];
    const int sl = (wc * 64 + lane) * N;
    if (RW > 1) {
#pragma unroll
        for (int e = 0; e < N; ++e) {
            sv[wr][sl + e] = acc[e].v;
            if (EXTREMUM(IS_MAX)) si[wr][sl + e] = acc[e].i;
        }
        __syncthreads();
    }
    if (wr == 0 && col < inner) {
#pragma unroll
        for (int e = 0; e < N; ++e) {
            Acc<T, IS_MAX> r = acc[e];
            for (int w = 1; w < RW; ++w) r.merge(sv[w][sl + e], EXTREMUM(IS_MAX) ? si[w][sl + e] : NO_INDEX);
            const i64 slot = (o * S + s) * inner + col + e;
            out[slot] = EXTREMUM(IS_MAX) ? r.v : r.v * scale;
            if (EXTREMUM(IS_MAX) && idx_out) idx_out[slot] = (final_pass && r.i == NO_INDEX) ? 0 : r.i;
        }
    }
}

template <typename T, int IS_MAX, bool VEC, int CW, bool STREAM>
void launch_col(fx_ctx* c, dim3 grid, const T* in, T* out, i64* idx_out, i64 axis, i64 inner, i64 chunk, T scale, int final_pass) {
    col_reduce_kernel<T, IS_MAX, VEC, false, CW, STREAM><<<grid, dim3(256), 0, c->stream>>>(in, nullptr, out, idx_out, axis, inner, chunk, scale, final_pass);
}

// Where the slice partials of a split reduction live: the context's growing scratch allocation, or, for the entry
// point that must not allocate, a fixed region of `fixed_bytes` (a request beyond it is refused).
struct PartialSpace {
    char* fixed = nullptr;
    i64 fixed_bytes = 0;
    // returns nullptr with the error message and *rc set
    char* get(fx_ctx* c, i64 bytes, const char* what, int* rc) const {
        if (fixed) {
            if (bytes > fixed_bytes) {
                fx::set_error("%s: this shape needs %lld bytes of slice partials, the fixed scratch holds %lld", what,
                              (long long)bytes, (long long)fixed_bytes);
                *rc = FX_ERR_UNSUPPORTED;
                return nullptr;
            }
            return fixed;
        }
        char* p = (char*)c->get_scratch(bytes);
        if (!p) *rc = FX_ERR_OOM;
        return p;
    }
};

template <typename T, int IS_MAX>
int reduce(fx_ctx* c, const T* in, T* out, i64* idx_out, i64 outer, i64 axis, i64 inner, T scale, const char* what,
           const PartialSpace& space = PartialSpace()) {
    if constexpr (IS_MAX == 1 || IS_MAX == 2) {
        // no position wanted: the value-only accumulator (same values; the scale of an extremum is 1)
        if (idx_out == nullptr) return reduce<T, IS_MAX + 3>(c, in, out, nullptr, outer, axis, inner, T(1), what, space);
    }
    FX_CHECK_CTX(c);
    FX_REQUIRE(outer >= 0 && axis >= 1 && inner >= 0, "%s: bad view [%lld, %lld, %lld]", what, (long long)outer,
               (long long)axis, (long long)inner);
    if (outer == 0 || inner == 0) return FX_OK;
    FX_REQUIRE(in && out, "%s: null pointer", what);
    FX_REQUIRE(outer <= 65535 * 1024ll, "%s: outer too large", what);
    constexpr int N = Vec16<T>::N;
    const bool want_idx = EXTREMUM(IS_MAX) && idx_out != nullptr;
    std::lock_guard<std::mutex> lk(c->launch_mutex);
    const i64 target_blocks = (i64)c->num_cus * 8;

    if (inner == 1) {
        if (axis % N == 0 && axis / N <= 64 && fx::aligned16(in)) {
            const int axis_v = (int)(axis / N);
            int GV = 1;
            while (GV < axis_v) GV <<= 1;
            const i64 blocks = fx::ceil_div(outer, (i64)4 * (256 / GV));
            FX_REQUIRE(blocks <= 0x7fffffff, "%s: too many rows", what);
            short_row_vec_kernel<T, IS_MAX><<<dim3((unsigned)blocks), dim3(256), 0, c->stream>>>(in, out, idx_out, outer, axis_v, GV, scale);
            FX_LAUNCH_CHECK();
            return FX_OK;
        }
        if (axis <= 64 && outer >= 1) {
            int G = 1;
            while (G < axis) G <<= 1;
            const i64 rows_per_block = 256 / G;
            const i64 blocks = fx::ceil_div(outer, rows_per_block);
            FX_REQUIRE(blocks <= 0x7fffffff, "%s: too many rows", what);
            short_row_reduce_kernel<T, IS_MAX><<<dim3((unsigned)blocks), dim3(256), 0, c->stream>>>(in, out, idx_out, outer, axis, G, scale);
            FX_LAUNCH_CHECK();
            return FX_OK;
        }
        FX_REQUIRE(outer <= 65535, "%s: more than 65535 long rows; reshape so that the reduced axis is not the last", what);
        // slices: enough blocks to fill the chip, each at least 16 KiB, slice length a multiple of 1024 elements
        i64 S = 1;
        const i64 row_want = (i64)c->num_cus * 3;  // measured on 2^26 elements: 2-4 blocks per CU is fastest
        if (outer < row_want) {
            S = std::min<i64>(fx::ceil_div(row_want, outer), std::max<i64>(1, axis / 4096));
            S = std::min<i64>(S, 65535);
        }
        i64 chunk = fx::ceil_div(axis, S);
        chunk = fx::ceil_div(chunk, 1024) * 1024;
        S = fx::ceil_div(axis, chunk);
        const bool vec = fx::aligned16(in) && (axis % N == 0);
        T* pv = out;
        i64* pi = idx_out;
        if (S > 1) {
            const i64 bytes = outer * S * (i64)(sizeof(T) + sizeof(i64));
            int rc = FX_OK;
            char* sc = space.get(c, bytes, what, &rc);
            if (!sc) return rc;
            pi = (i64*)sc;
            pv = (T*)(sc + outer * S * sizeof(i64));
        }
        const dim3 grid((unsigned)S, (unsigned)outer), block(256);
        const T sc1 = S > 1 ? T(1) : scale;
        i64* io = (S > 1 && EXTREMUM(IS_MAX)) ? pi : idx_out;
        const bool stream = outer * axis * (i64)sizeof(T) >= STREAM_BYTES;
        if (vec && stream) row_reduce_kernel<T, IS_MAX, true, true><<<grid, block, 0, c->stream>>>(in, pv, io, axis, chunk, sc1);
        else if (vec) row_reduce_kernel<T, IS_MAX, true, false><<<grid, block, 0, c->stream>>>(in, pv, io, axis, chunk, sc1);
        else row_reduce_kernel<T, IS_MAX, false, false><<<grid, block, 0, c->stream>>>(in, pv, io, axis, chunk, sc1);
        FX_LAUNCH_CHECK();
        if (S > 1) {
            combine_rows_kernel<T, IS_MAX><<<dim3((unsigned)outer), dim3(256), 0, c->stream>>>(
                pv, EXTREMUM(IS_MAX) ? pi : nullptr, out, idx_out, outer, S, scale);
            FX_LAUNCH_CHECK();
        }
        (void)want_idx;
        return FX_OK;
    }

    // column reduction
    FX_REQUIRE(outer <= 65535, "%s: outer %lld exceeds 65535 for a column reduction", what, (long long)outer);
    const bool vec = fx::aligned16(in) && (inner % N == 0);
    const bool stream = outer * axis * inner * (i64)sizeof(T) >= STREAM_BYTES;
    const int NV = vec ? N : 1;
    const bool wide = vec && inner >= 4 * 64 * NV;  // four waves side by side: 4 KiB contiguous per row and block
    const i64 cols_per_block = (wide ? 4 : 1) * 64 * NV;
    const i64 tiles = fx::ceil_div(inner, cols_per_block);
    FX_REQUIRE(tiles <= 0x7fffffff, "%s: inner too large", what);
    i64 S = 1;
    // measured on [8192,8192]: about 0.75 blocks per CU (each keeping 32 KiB of loads in flight) is fastest
    const i64 want = wide ? (i64)c->num_cus * 3 / 4 : target_blocks;
    if (tiles * outer < want) {
        S = std::min<i64>(fx::ceil_div(want, tiles * outer), std::max<i64>(1, axis / 32));
        S = std::min<i64>(S, 65535);
    }
    i64 chunk = fx::ceil_div(axis, S);
    chunk = fx::ceil_div(chunk, 4) * 4;
    S = fx::ceil_div(axis, chunk);
    T* pv = out;
    i64* pi = idx_out;
    if (S > 1) {
        const i64 n_part = outer * S * inner;
        const i64 bytes = n_part * (i64)(sizeof(T) + (EXTREMUM(IS_MAX) ? sizeof(i64) : 0)) + 256;
        int rc = FX_OK;
        char* sc = space.get(c, bytes, what, &rc);
        if (!sc) return rc;
        pi = EXTREMUM(IS_MAX) ? (i64*)sc : nullptr;
        pv = (T*)(sc + (EXTREMUM(IS_MAX) ? ((n_part * sizeof(i64) + 255) / 256) * 256 : 0));
    }
    {
        const dim3 grid((unsigned)tiles, (unsigned)S, (unsigned)outer);
        const T sc1 = S > 1 ? T(1) : scale;
        const int fin = S > 1 ? 0 : 1;
        if (wide && stream) launch_col<T, IS_MAX, true, 4, true>(c, grid, in, pv, pi, axis, inner, chunk, sc1, fin);
        else if (wide) launch_col<T, IS_MAX, true, 4, false>(c, grid, in, pv, pi, axis, inner, chunk, sc1, fin);
        else if (vec) launch_col<T, IS_MAX, true, 1, false>(c, grid, in, pv, pi, axis, inner, chunk, sc1, fin);
        else launch_col<T, IS_MAX, false, 1, false>(c, grid, in, pv, pi, axis, inner, chunk, sc1, fin);
        FX_LAUNCH_CHECK();
    }
    if (S > 1) {
        // second pass over [outer, S, inner] partials; scalar columns so that many blocks share the work
        const i64 tiles2 = fx::ceil_div(inner, 64);
        const dim3 grid((unsigned)tiles2, 1, (unsigned)outer), block(256);
        col_reduce_kernel<T, IS_MAX, false, true, 1, false><<<grid, block, 0, c->stream>>>(pv, pi, out, idx_out, S, inner, fx::ceil_div(S, 4) * 4, scale, 1);
        FX_LAUNCH_CHECK();
    }
    return FX_OK;
}

// ---- softmax over the middle axis: cpu.rs:1037-1068 -----------------------------------------------------
template <typename T> __device__ __forceinline__ T dev_exp(T x);
template <> __device__ __forceinline__ float dev_exp<float>(float x) { return expf(x); }
template <> __device__ __forceinline__ double dev_exp<double>(double x) { return exp(x); }

template <typename T>
__global__ __launch_bounds__(256) void softmax_axis_kernel(const T* __restrict__ in, T* __restrict__ out, i64 outer, i64 axis, i64 inner) {
    const i64 t = (i64)blockIdx.x * 256 + threadIdx.x;
    if (t >= outer * inner) return;
    const i64 o = t / inner, i = t - o * inner;
    const T* p = in + o * axis * inner + i;
    T* q = out + o * axis * inner + i;
    T m = lowest<T>();
    for (i64 a = 0; a < axis; ++a) { const T x = p[a * inner]; if (x > m) m = x; }
    T s = T(0);
    for (i64 a = 0; a < axis; ++a) { const T e = dev_exp<T>(p[a * inner] - m); q[a * inner] = e; s = s + e; }
    for (i64 a = 0; a < axis; ++a) q[a * inner] = q[a * inner] / s;
}

// Long contiguous rows (inner == 1, e.g. the whole-tensor softmax of cpu.rs:1018-1036 viewed as one row): one block per
// row; maximum, sum of exponentials and the division each run block-wide.  The sum is a fixed tree (reproducible),
// not the one-thread running sum of the kernel above.
template <typename T>
__global__ __launch_bounds__(256) void softmax_row_kernel(const T* __restrict__ in, T* __restrict__ out, i64 axis) {
    __shared__ T sm[256];
    const T* p = in + (i64)blockIdx.x * axis;
    T* q = out + (i64)blockIdx.x * axis;
    T m = lowest<T>();
    for (i64 a = threadIdx.x; a < axis; a += 256) { const T x = p[a]; if (x > m) m = x; }
    sm[threadIdx.x] = m;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) {
        if ((int)threadIdx.x < w && sm[threadIdx.x + w] > sm[threadIdx.x]) sm[threadIdx.x] = sm[threadIdx.x + w];
        __syncthreads();
    }
    m = sm[0];
    __syncthreads();
    T s = T(0);
    for (i64 a = threadIdx.x; a < axis; a += 256) { const T e = dev_exp<T>(p[a] - m); q[a] = e; s = s + e; }
    sm[threadIdx.x] = s;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) {
        if ((int)threadIdx.x < w) sm[threadIdx.x] = sm[threadIdx.x] + sm[threadIdx.x + w];
        __syncthreads();
    }
    s = sm[0];
    for (i64 a = threadIdx.x; a < axis; a += 256) q[a] = q[a] / s;
}

template <typename T>
int softmax_axis(fx_ctx* c, const T* in, T* out, i64 outer, i64 axis, i64 inner) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(outer >= 0 && axis >= 1 && inner >= 0, "fx_softmax_axis: bad view");
    if (outer == 0 || inner == 0) return FX_OK;
    FX_REQUIRE(in && out, "fx_softmax_axis: null pointer");
    FX_REQUIRE(in != out, "fx_softmax_axis: in-place not supported");
    if (inner == 1 && axis >= 2048 && outer <= 0x7fffffff) {
        softmax_row_kernel<T><<<dim3((unsigned)outer), dim3(256), 0, c->stream>>>(in, out, axis);
        FX_LAUNCH_CHECK();
        return FX_OK;
    }
    const i64 blocks = fx::ceil_div(outer * inner, 256);
    FX_REQUIRE(blocks <= 0x7fffffff, "fx_softmax_axis: too many rows");
    softmax_axis_kernel<T><<<dim3((unsigned)blocks), dim3(256), 0, c->stream>>>(in, out, outer, axis, inner);
    FX_LAUNCH_CHECK();
    return FX_OK;
}

}  // namespace

// ---- the entry point that allocates nothing ---------------------------------------------------------------
// Slice partials of fx_reduce_max_noalloc_f32 live in this array instead of the context's hipMalloc'ed scratch.
// Every device the library is loaded on holds its own copy at its own address; host code uses the address
// hipGetSymbolAddress returned for the device, never the array's name.
static __device__ __align__(256) unsigned char scratch[FX_NOALLOC_SCRATCH_BYTES];

namespace fx {
constexpr int MAX_DEVICES = 64;
static char* g_static_scratch[MAX_DEVICES] = {};
static std::mutex g_static_scratch_mutex;
// Called by fx_init with `device` current: resolves this device's copy of the array once.
int static_scratch_init(int device) {
    if (device < 0 || device >= MAX_DEVICES) return FX_OK;  // the no-alloc entry point refuses such a device itself
    std::lock_guard<std::mutex> lk(g_static_scratch_mutex);
    if (g_static_scratch[device]) return FX_OK;
    void* p = nullptr;
    FX_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    g_static_scratch[device] = (char*)p;
    return FX_OK;
}
}  // namespace fx

extern "C" int fx_reduce_max_noalloc_f32(fx_ctx* c, const float* in, float* out, int64_t* idx, int64_t outer, int64_t axis,
                                         int64_t inner) {
    FX_REQUIRE(c != nullptr, "null context");
    FX_REQUIRE(c->device >= 0 && c->device < fx::MAX_DEVICES && fx::g_static_scratch[c->device] != nullptr,
               "fx_reduce_max_noalloc: no fixed scratch was resolved for device %d", c->device);
    PartialSpace space;
    space.fixed = fx::g_static_scratch[c->device];
    space.fixed_bytes = FX_NOALLOC_SCRATCH_BYTES;
    return reduce<float, 1>(c, in, out, idx, outer, axis, inner, 1.0f, "fx_reduce_max_noalloc", space);
}

#define FX_DEFINE_REDUCE(T, S)                                                                                         \
    extern "C" int fx_reduce_sum_##S(fx_ctx* c, const T* in, T* out, int64_t outer, int64_t axis, int64_t inner) {     \
        return reduce<T, false>(c, in, out, nullptr, outer, axis, inner, T(1), "fx_reduce_sum");                       \
    }                                                                                                                  \
    extern "C" int fx_reduce_mean_##S(fx_ctx* c, const T* in, T* out, int64_t outer, int64_t axis, int64_t inner) {    \
        FX_REQUIRE(axis >= 1, "fx_reduce_mean: empty axis");                                                           \
        return reduce<T, false>(c, in, out, nullptr, outer, axis, inner, (T)(1.0 / (double)axis), "fx_reduce_mean");   \
    }                                                                                                                  \
    extern "C" int fx_reduce_max_##S(fx_ctx* c, const T* in, T* out, int64_t* idx, int64_t outer, int64_t axis,        \
                                     int64_t inner) {                                                                  \
        return reduce<T, 1>(c, in, out, idx, outer, axis, inner, T(1), "fx_reduce_max");                               \
    }                                                                                                                  \
    extern "C" int fx_reduce_min_##S(fx_ctx* c, const T* in, T* out, int64_t* idx, int64_t outer, int64_t axis,        \
                                     int64_t inner) {                                                                  \
        return reduce<T, 2>(c, in, out, idx, outer, axis, inner, T(1), "fx_reduce_min");                               \
    }                                                                                                                  \
    extern "C" int fx_reduce_prod_##S(fx_ctx* c, const T* in, T* out, int64_t outer, int64_t axis, int64_t inner) {    \
        return reduce<T, 3>(c, in, out, nullptr, outer, axis, inner, T(1), "fx_reduce_prod");                          \
    }                                                                                                                  \
    extern "C" int fx_softmax_axis_##S(fx_ctx* c, const T* in, T* out, int64_t outer, int64_t axis, int64_t inner) {   \
        return softmax_axis<T>(c, in, out, outer, axis, inner);                                                        \
    }

FX_DEFINE_REDUCE(float, f32)
FX_DEFINE_REDUCE(double, f64)
