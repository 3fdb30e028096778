// Elementwise kernels (binary, scalar, unary, clamp, fill, fused activation gradients, materialize).
// Replaces kernels/elementwise.cu, activations.cu (relu/sigmoid/tanh), comparison.cu, fill.cu, materialize.cu
// of the reference with wave64 streaming kernels: 16-byte vector accesses, four independent vectors in flight per
// thread, one pass over memory.  HBM-bound: 2 or 3 arrays of n elements per call.
// Built with floating-point contraction off so composed expressions round op by op like the CPU backend.
#include "common.hpp"

namespace {

template <typename T> struct Vec16;
template <> struct Vec16<float> { typedef float4 type; static constexpr int N = 4; };
template <> struct Vec16<double> { typedef double2 type; static constexpr int N = 2; };

template <typename T> __device__ __forceinline__ T vget(const typename Vec16<T>::type& v, int i);
template <> __device__ __forceinline__ float vget<float>(const float4& v, int i) { return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w; }
template <> __device__ __forceinline__ double vget<double>(const double2& v, int i) { return i == 0 ? v.x : v.y; }
template <typename T> __device__ __forceinline__ void vset(typename Vec16<T>::type& v, int i, T x);
template <> __device__ __forceinline__ void vset<float>(float4& v, int i, float x) { if (i == 0) v.x = x; else if (i == 1) v.y = x; else if (i == 2) v.z = x; else v.w = x; }
template <> __device__ __forceinline__ void vset<double>(double2& v, int i, double x) { if (i == 0) v.x = x; else v.y = x; }

constexpr int EW_THREADS = 256;
constexpr int EW_UNROLL = 4;
constexpr i64 EW_STREAM_BYTES = 128ll << 20;  // arrays at least this large are streamed past the caches

typedef float nt_f4 __attribute__((ext_vector_type(4)));
typedef double nt_d2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float4 nt_load(const float4* p) { const nt_f4 v = __builtin_nontemporal_load(reinterpret_cast<const nt_f4*>(p)); return float4{v.x, v.y, v.z, v.w}; }
__device__ __forceinline__ double2 nt_load(const double2* p) { const nt_d2 v = __builtin_nontemporal_load(reinterpret_cast<const nt_d2*>(p)); return double2{v.x, v.y}; }
__device__ __forceinline__ void nt_store(float4 r, float4* p) { const nt_f4 v = {r.x, r.y, r.z, r.w}; __builtin_nontemporal_store(v, reinterpret_cast<nt_f4*>(p)); }
__device__ __forceinline__ void nt_store(double2 r, double2* p) { const nt_d2 v = {r.x, r.y}; __builtin_nontemporal_store(v, reinterpret_cast<nt_d2*>(p)); }

// NIN = number of input arrays (0, 1 or 2).  F: T operator()(T a, T b).
// Cached variant (small arrays: the consumer kernel finds the data in L2 / Infinity Cache): four 16-byte vectors in
// flight per thread.
template <typename T, int NIN, class F>
__global__ __launch_bounds__(EW_THREADS) void ew_vec_kernel(const T* __restrict__ a, const T* __restrict__ b,
                                                            T* __restrict__ out, i64 nvec, F f) {
    typedef typename Vec16<T>::type V;
    constexpr int N = Vec16<T>::N;
    const V* av = reinterpret_cast<const V*>(a);
    const V* bv = reinterpret_cast<const V*>(b);
    V* ov = reinterpret_cast<V*>(out);
    const i64 base = (i64)blockIdx.x * (EW_THREADS * EW_UNROLL) + threadIdx.x;
    V ra[EW_UNROLL], rb[EW_UNROLL];
#pragma unroll
    for (int j = 0; j < EW_UNROLL; ++j) {
        const i64 i = base + (i64)j * EW_THREADS;
        if (i < nvec) {
            if (NIN >= 1) ra[j] = av[i];
            if (NIN >= 2) rb[j] = bv[i];
        }
    }
#pragma unroll
    for (int j = 0; j < EW_UNROLL; ++j) {
        const i64 i = base + (i64)j * EW_THREADS;
        if (i < nvec) {
            V r;
#pragma unroll
            for (int e = 0; e < N; ++e)
                vset<T>(r, e, f(NIN >= 1 ? vget<T>(ra[j], e) : T(0), NIN >= 2 ? vget<T>(rb[j], e) : T(0)));
            ov[i] = r;
        }
    }
}

// Streaming variant (large arrays): one 16-byte vector per thread, non-temporal loads and stores, many small waves.
// Measured on MI355X for c = a + b over 2^28 floats: 6.4 TB/s against 5.65 TB/s for the cached variant.
template <typename T, int NIN, class F>
__global__ __launch_bounds__(EW_THREADS) void ew_stream_kernel(const T* __restrict__ a, const T* __restrict__ b,
                                                               T* __restrict__ out, i64 nvec, F f) {
    typedef typename Vec16<T>::type V;
    constexpr int N = Vec16<T>::N;
    const i64 i = (i64)blockIdx.x * EW_THREADS + threadIdx.x;
    if (i >= nvec) return;
    V ra, rb;
    if (NIN >= 1) ra = nt_load(reinterpret_cast<const V*>(a) + i);
    if (NIN >= 2) rb = nt_load(reinterpret_cast<const V*>(b) + i);
    V r;
#pragma unroll
    for (int e = 0; e < N; ++e) vset<T>(r, e, f(NIN >= 1 ? vget<T>(ra, e) : T(0), NIN >= 2 ? vget<T>(rb, e) : T(0)));
    nt_store(r, reinterpret_cast<V*>(out) + i);
}

template <typename T, int NIN, class F>
__global__ __launch_bounds__(EW_THREADS) void ew_scalar_kernel(const T* __restrict__ a, const T* __restrict__ b,
                                                               T* __restrict__ out, i64 begin, i64 n, F f) {
    const i64 i = begin + (i64)blockIdx.x * EW_THREADS + threadIdx.x;
    if (i < n) out[i] = f(NIN >= 1 ? a[i] : T(0), NIN >= 2 ? b[i] : T(0));
}

template <typename T, int NIN, class F>
int launch_ew(fx_ctx* c, const T* a, const T* b, T* out, i64 n, F f, const char* what) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(n >= 0, "%s: negative element count", what);
    if (n == 0) return FX_OK;
    FX_REQUIRE(out != nullptr && (NIN < 1 || a != nullptr) && (NIN < 2 || b != nullptr), "%s: null pointer", what);
    constexpr int N = Vec16<T>::N;
    const bool vec_ok = fx::aligned16(out) && (NIN < 1 || fx::aligned16(a)) && (NIN < 2 || fx::aligned16(b));
    i64 done = 0;
    if (vec_ok && n >= N) {
        const i64 nvec = n / N;
        if (n * (i64)sizeof(T) >= EW_STREAM_BYTES) {
            const i64 blocks = fx::ceil_div(nvec, (i64)EW_THREADS);
            FX_REQUIRE(blocks <= 0x7fffffff, "%s: too many elements", what);
            ew_stream_kernel<T, NIN, F><<<dim3((unsigned)blocks), dim3(EW_THREADS), 0, c->stream>>>(a, b, out, nvec, f);
        } else {
            const i64 blocks = fx::ceil_div(nvec, (i64)EW_THREADS * EW_UNROLL);
            ew_vec_kernel<T, NIN, F><<<dim3((unsigned)blocks), dim3(EW_THREADS), 0, c->stream>>>(a, b, out, nvec, f);
        }
        FX_LAUNCH_CHECK();
        done = nvec * N;
    }
    if (done < n) {
        const i64 blocks = fx::ceil_div(n - done, (i64)EW_THREADS);
        FX_REQUIRE(blocks <= 0x7fffffff, "%s: too many elements", what);
        ew_scalar_kernel<T, NIN, F><<<dim3((unsigned)blocks), dim3(EW_THREADS), 0, c->stream>>>(a, b, out, done, n, f);
        FX_LAUNCH_CHECK();
    }
    return FX_OK;
}

// ---- functors -------------------------------------------------------------------------------------------
template <typename T> __device__ __forceinline__ T dev_exp(T x);
template <> __device__ __forceinline__ float dev_exp<float>(float x) { return expf(x); }
template <> __device__ __forceinline__ double dev_exp<double>(double x) { return exp(x); }
template <typename T> __device__ __forceinline__ T dev_log(T x);
template <> __device__ __forceinline__ float dev_log<float>(float x) { return logf(x); }
template <> __device__ __forceinline__ double dev_log<double>(double x) { return log(x); }
template <typename T> __device__ __forceinline__ T dev_sqrt(T x);
template <> __device__ __forceinline__ float dev_sqrt<float>(float x) { return sqrtf(x); }
template <> __device__ __forceinline__ double dev_sqrt<double>(double x) { return sqrt(x); }

template <typename T> __device__ __forceinline__ T dev_pow(T x, T y);
template <> __device__ __forceinline__ float dev_pow<float>(float x, float y) { return powf(x, y); }
template <> __device__ __forceinline__ double dev_pow<double>(double x, double y) { return pow(x, y); }

template <typename T, int OP> struct BinF {
    __device__ __forceinline__ T operator()(T x, T y) const {
        if (OP == FX_ADD) return x + y;
        if (OP == FX_SUB) return x - y;
        if (OP == FX_MUL) return x * y;
        if (OP == FX_DIV) return x / y;
        if (OP == FX_EQUAL) return x == y ? T(1) : T(0);
        if (OP == FX_GREATER) return x > y ? T(1) : T(0);
        if (OP == FX_GREATER_EQUAL) return x >= y ? T(1) : T(0);
        if (OP == FX_LESS) return x < y ? T(1) : T(0);
        if (OP == FX_LESS_EQUAL) return x <= y ? T(1) : T(0);
        if (OP == FX_MIN) return x <= y ? x : y;
        if (OP == FX_POW) return dev_pow<T>(x, y);
        return x >= y ? x : y;  // FX_MAX
    }
};

template <typename T, int OP> struct ScalarF {
    T s;
    __device__ __forceinline__ T operator()(T x, T) const {
        if (OP == FX_ADD_SCALAR) return x + s;
        if (OP == FX_SUB_SCALAR) return x - s;
        if (OP == FX_MUL_SCALAR) return x * s;
        if (OP == FX_DIV_SCALAR) return x / s;
        if (OP == FX_GREATER_SCALAR) return x > s ? T(1) : T(0);
        if (OP == FX_GREATER_EQUAL_SCALAR) return x >= s ? T(1) : T(0);
        if (OP == FX_LESS_EQUAL_SCALAR) return x <= s ? T(1) : T(0);
        if (OP == FX_POW_SCALAR) return dev_pow<T>(x, s);
        return x < s ? T(1) : T(0);  // FX_LESS_SCALAR
    }
};

// tanh with the CPU backend's branches (cpu.rs:1108-1147)
template <typename T> __device__ __forceinline__ T tanh_like_cpu(T x) {
    if (x > T(20)) return T(1);
    if (x < T(-20)) return T(-1);
    if (x >= T(0)) {
        const T e = dev_exp<T>(-x * T(2));
        const T num = T(1) - e, den = T(1) + e;
        return den == T(0) ? T(1) : num / den;
    }
    const T e = dev_exp<T>(x * T(2));
    const T num = e - T(1), den = e + T(1);
    return den == T(0) ? T(-1) : num / den;
}

template <typename T, int OP> struct UnaryF {
    __device__ __forceinline__ T operator()(T x, T) const {
        if (OP == FX_NEG) return -x;
        if (OP == FX_SQRT) return dev_sqrt<T>(x);
        if (OP == FX_EXP) return dev_exp<T>(x);
        if (OP == FX_LOG) return dev_log<T>(x);
        if (OP == FX_RELU) return x > T(0) ? x : T(0);
        if (OP == FX_SIGMOID) return T(1) / (T(1) + dev_exp<T>(-x));
        if (OP == FX_TANH) return tanh_like_cpu<T>(x);
        if (OP == FX_ABS) return x < T(0) ? -x : x;
        if (OP == FX_SIGN) return x > T(0) ? T(1) : (x < T(0) ? T(-1) : T(0));
        if (OP == FX_LOGICAL_NOT) return x == T(0) ? T(1) : T(0);
        return T(1) / x;  // FX_RECIPROCAL
    }
};

template <typename T> struct ClampF {
    T lo, hi;
    __device__ __forceinline__ T operator()(T x, T) const { return x < lo ? lo : (x > hi ? hi : x); }
};
template <typename T> struct InRangeF {
    T lo, hi;
    __device__ __forceinline__ T operator()(T x, T) const { return (x >= lo && x <= hi) ? T(1) : T(0); }
};
template <typename T> struct CopyF {  // moves the bits: no arithmetic touches the value
    __device__ __forceinline__ T operator()(T x, T) const { return x; }
};
template <typename T> struct FillF {
    T v;
    __device__ __forceinline__ T operator()(T, T) const { return v; }
};
template <typename T> struct ReluBwdF {  // (g, x)
    __device__ __forceinline__ T operator()(T g, T x) const { return g * (x > T(0) ? T(1) : T(0)); }
};
template <typename T, int LITERAL> struct SigmoidBwdF {  // (g, s)
    __device__ __forceinline__ T operator()(T g, T s) const {
        const T t = LITERAL ? (s - T(1)) : (T(1) - s);
        const T local = s * t;
        return g * local;
    }
};
template <typename T> struct TanhBwdF {  // (g, t)
    __device__ __forceinline__ T operator()(T g, T t) const {
        const T sq = t * t;
        const T m = sq - T(1);
        return g * (-m);
    }
};

template <typename T>
int binary_dispatch(fx_ctx* c, int op, const T* a, const T* b, T* o, i64 n) {
    switch (op) {
#define CASE(OP) case OP: return launch_ew<T, 2>(c, a, b, o, n, BinF<T, OP>{}, "fx_binary");
        CASE(FX_ADD) CASE(FX_SUB) CASE(FX_MUL) CASE(FX_DIV) CASE(FX_EQUAL) CASE(FX_GREATER) CASE(FX_GREATER_EQUAL)
        CASE(FX_LESS) CASE(FX_LESS_EQUAL) CASE(FX_MIN) CASE(FX_MAX) CASE(FX_POW)
#undef CASE
    }
    fx::set_error("fx_binary: unknown op %d", op);
    return FX_ERR_INVALID;
}

template <typename T>
int scalar_dispatch(fx_ctx* c, int op, const T* a, T s, T* o, i64 n) {
    switch (op) {
#define CASE(OP) case OP: return launch_ew<T, 1>(c, a, (const T*)nullptr, o, n, ScalarF<T, OP>{s}, "fx_scalar");
        CASE(FX_ADD_SCALAR) CASE(FX_SUB_SCALAR) CASE(FX_MUL_SCALAR) CASE(FX_DIV_SCALAR) CASE(FX_GREATER_SCALAR)
        CASE(FX_GREATER_EQUAL_SCALAR) CASE(FX_LESS_EQUAL_SCALAR) CASE(FX_LESS_SCALAR) CASE(FX_POW_SCALAR)
#undef CASE
    }
    fx::set_error("fx_scalar: unknown op %d", op);
    return FX_ERR_INVALID;
}

template <typename T>
int unary_dispatch(fx_ctx* c, int op, const T* a, T* o, i64 n) {
    switch (op) {
#define CASE(OP) case OP: return launch_ew<T, 1>(c, a, (const T*)nullptr, o, n, UnaryF<T, OP>{}, "fx_unary");
        CASE(FX_NEG) CASE(FX_SQRT) CASE(FX_EXP) CASE(FX_LOG) CASE(FX_RELU) CASE(FX_SIGMOID) CASE(FX_TANH) CASE(FX_ABS)
        CASE(FX_RECIPROCAL) CASE(FX_SIGN) CASE(FX_LOGICAL_NOT)
#undef CASE
    }
    fx::set_error("fx_unary: unknown op %d", op);
    return FX_ERR_INVALID;
}

// ---- materialize: gather a strided / broadcast view into contiguous memory ------------------------------
struct ViewDesc {
    int ndim;
    i64 shape[8];
    i64 stride[8];
};

template <typename T>
__global__ __launch_bounds__(256) void materialize_kernel(const T* __restrict__ in, T* __restrict__ out, ViewDesc v, i64 n) {
    const i64 i = (i64)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    i64 r = i, off = 0;
#pragma unroll
    for (int d = 7; d >= 0; --d) {
        if (d < v.ndim) {
            const i64 q = r / v.shape[d];
            off += (r - q * v.shape[d]) * v.stride[d];
            r = q;
        }
    }
    out[i] = in[off];
}

// Collapsed view of at most 4 dims whose innermost dim is contiguous (stride 1) or broadcast (stride 0) with an
// extent that is a multiple of the 16-byte vector: 32-bit index arithmetic with multiply-shift division.
struct U32Div {
    uint32_t d, m, s;
    __device__ __forceinline__ uint32_t div(uint32_t n) const { return (uint32_t)(((uint64_t)__umulhi(n, m) + n) >> s); }
};
static U32Div make_u32div(uint32_t d) {
    U32Div r;
    r.d = d;
    r.s = 0;
    while ((1ull << r.s) < d) ++r.s;
    r.m = (uint32_t)((((1ull << 32) * ((1ull << r.s) - d)) / d) + 1);
    return r;
}
struct FastView {
    U32Div inner4;      // vectors along the innermost dim
    int inner_stride;   // 0 or 1
    U32Div ext[3];      // outer dims, innermost of them first (extent 1 when absent)
    i64 stride[3];
};

struct CollapsedView {
    int nd;
    U32Div ext[8];  // innermost first
    i64 stride[8];
};

// Any collapsed view below 2^31 elements, one element per thread.
template <typename T>
__global__ __launch_bounds__(256) void materialize_u32_kernel(const T* __restrict__ in, T* __restrict__ out, CollapsedView v, i64 n) {
    const i64 i = (i64)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    uint32_t r = (uint32_t)i;
    i64 off = 0;
#pragma unroll
    for (int d = 0; d < 8; ++d) {
        if (d < v.nd) {
            const uint32_t q = v.ext[d].div(r);
            off += (i64)(r - q * v.ext[d].d) * v.stride[d];
            r = q;
        }
    }
    out[i] = in[off];
}

template <typename T, bool SRC_VEC>
__global__ __launch_bounds__(256) void materialize_vec_kernel(const T* __restrict__ in, T* __restrict__ out, FastView v, i64 nv) {
    constexpr int V = 16 / (int)sizeof(T);
    typedef T vec_t __attribute__((ext_vector_type(V)));
    const i64 i = (i64)blockIdx.x * 256 + threadIdx.x;
    if (i >= nv) return;
    uint32_t r = (uint32_t)i;
    uint32_t q = v.inner4.div(r);
    i64 off = (i64)(r - q * v.inner4.d) * V * v.inner_stride;
    r = q;
#pragma unroll
    for (int d = 0; d < 3; ++d) {
        q = v.ext[d].div(r);
        off += (i64)(r - q * v.ext[d].d) * v.stride[d];
        r = q;
    }
    vec_t o;
    if (SRC_VEC) {
        o = *reinterpret_cast<const vec_t*>(in + off);
    } else if (v.inner_stride == 0) {
        const T x = in[off];
#pragma unroll
        for (int u = 0; u < V; ++u) o[u] = x;
    } else {
#pragma unroll
        for (int u = 0; u < V; ++u) o[u] = in[off + u];
    }
    *reinterpret_cast<vec_t*>(out + i * V) = o;
}

// Transposed innermost pair: out[b][i][j] = in[b*sb + i + j*ld] (the view a 2-D transpose, or a batch of them, leaves
// behind).  64 x 64 tiles through LDS so that both the reads (along i) and the writes (along j) are contiguous;
// the 65-float pitch keeps the column reads of the tile on distinct banks.
template <typename T>
__global__ __launch_bounds__(256) void transpose_tile_kernel(const T* __restrict__ in, T* __restrict__ out, i64 I, i64 J, i64 ld, i64 sb) {
    __shared__ T tile[64][65];
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    // diagonal order: the blocks that run together read source rows of different tile columns, so a power-of-two pitch does
    // not send all of them to the same memory channels
    const i64 j0 = (i64)((blockIdx.x + blockIdx.y) % gridDim.x) * 64, i0 = (i64)blockIdx.y * 64, b = blockIdx.z;
    const T* src = in + b * sb;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const i64 j = j0 + ty + 4 * r, i = i0 + tx;
        if (j < J && i < I) tile[ty + 4 * r][tx] = src[j * ld + i];
    }
    __syncthreads();
    T* dst = out + b * I * J;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const i64 i = i0 + ty + 4 * r, j = j0 + tx;
        if (i < I && j < J) dst[i * J + j] = tile[tx][ty + 4 * r];
    }
}

// The same tiles with 16-byte global accesses (both extents, the source pitch and the batch pitch multiples of the vector
// length, 16-byte aligned pointers): a thread moves V consecutive elements per access, the transposition happens in the LDS
// tile, whose reads and writes stay at two lanes per bank.
template <typename T>
__global__ __launch_bounds__(256) void transpose_tile_vec_kernel(const T* __restrict__ in, T* __restrict__ out, i64 I, i64 J, i64 ld, i64 sb) {
    constexpr int V = 16 / (int)sizeof(T), VPR = 64 / V, RPP = 256 / VPR;  // vectors per tile row, rows per pass
    typedef T vec_t __attribute__((ext_vector_type(V)));
    __shared__ T tile[64][65];
    const int vx = threadIdx.x % VPR, vy = threadIdx.x / VPR;
    // diagonal order: the blocks that run together read source rows of different tile columns, so a power-of-two pitch does
    // not send all of them to the same memory channels
    const i64 j0 = (i64)((blockIdx.x + blockIdx.y) % gridDim.x) * 64, i0 = (i64)blockIdx.y * 64, b = blockIdx.z;
    const T* src = in + b * sb;
#pragma unroll
    for (int r = 0; r < 64 / RPP; ++r) {
        const int jl = vy + RPP * r;
        const i64 j = j0 + jl, i = i0 + vx * V;
        if (j < J && i < I) {
            const vec_t v = *reinterpret_cast<const vec_t*>(src + j * ld + i);
#pragma unroll
            for (int e = 0; e < V; ++e) tile[jl][vx * V + e] = v[e];
        }
    }
    __syncthreads();
    T* dst = out + b * I * J;
#pragma unroll
    for (int r = 0; r < 64 / RPP; ++r) {
        const int il = vy + RPP * r;
        const i64 i = i0 + il, j = j0 + vx * V;
        if (i < I && j < J) {
            vec_t v;
#pragma unroll
            for (int e = 0; e < V; ++e) v[e] = tile[vx * V + e][il];
            *reinterpret_cast<vec_t*>(dst + i * J + j) = v;
        }
    }
}

template <typename T>
int materialize(fx_ctx* c, const T* in, T* out, const i64* shape, const i64* strides, int ndim, i64 n) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(ndim >= 0 && ndim <= 8, "fx_materialize: ndim %d not in 0..8", ndim);
    FX_REQUIRE(n >= 0, "fx_materialize: negative element count");
    if (n == 0) return FX_OK;
    FX_REQUIRE(in && out && (ndim == 0 || (shape && strides)), "fx_materialize: null pointer");
    ViewDesc v{};
    v.ndim = ndim;
    i64 prod = 1;
    for (int d = 0; d < ndim; ++d) {
        FX_REQUIRE(shape[d] > 0 && strides[d] >= 0, "fx_materialize: bad shape/stride at dim %d", d);
        v.shape[d] = shape[d];
        v.stride[d] = strides[d];
        prod *= shape[d];
    }
    FX_REQUIRE(prod == n, "fx_materialize: shape product %lld != n %lld", (long long)prod, (long long)n);
    // Collapse the view: drop extent-1 dims, merge neighbours that walk memory as one dim (or are both broadcast).
    i64 cs[8], ct[8];
    int nd = 0;
    for (int d = 0; d < ndim; ++d) {
        if (shape[d] == 1) continue;
        if (nd > 0 && ct[nd - 1] == strides[d] * shape[d]) {
            cs[nd - 1] *= shape[d];
            ct[nd - 1] = strides[d];
        } else {
            cs[nd] = shape[d];
            ct[nd] = strides[d];
            ++nd;
        }
    }
    constexpr int V = 16 / (int)sizeof(T);
    if ((nd == 2 || nd == 3) && ct[nd - 2] == 1 && ct[nd - 1] > 1 && cs[nd - 2] >= 16 && cs[nd - 1] >= 16) {
        const i64 I = cs[nd - 2], J = cs[nd - 1], Bn = nd == 3 ? cs[0] : 1;
        const i64 gx = fx::ceil_div(J, 64), gy = fx::ceil_div(I, 64);
        if (gx <= 0x7fffffff && gy <= 65535 && Bn <= 65535) {
            const i64 ld = ct[nd - 1], sb = nd == 3 ? ct[0] : 0;
            constexpr i64 VT = 16 / (i64)sizeof(T);
            if (I % VT == 0 && J % VT == 0 && ld % VT == 0 && sb % VT == 0 && (((uintptr_t)in | (uintptr_t)out) & 15) == 0)
                transpose_tile_vec_kernel<T><<<dim3((unsigned)gx, (unsigned)gy, (unsigned)Bn), dim3(256), 0, c->stream>>>(in, out, I, J, ld, sb);
            else
                transpose_tile_kernel<T><<<dim3((unsigned)gx, (unsigned)gy, (unsigned)Bn), dim3(256), 0, c->stream>>>(in, out, I, J, ld, sb);
            FX_LAUNCH_CHECK();
            return FX_OK;
        }
    }
    if (nd >= 1 && nd <= 4 && n < (1ll << 31) && cs[nd - 1] % V == 0 && (ct[nd - 1] == 0 || ct[nd - 1] == 1) &&
        ((uintptr_t)out & 15) == 0) {
        // vector path: one thread writes V consecutive outputs of the innermost collapsed dim
        bool src_vec = ct[nd - 1] == 1 && ((uintptr_t)in & 15) == 0;
        FastView fv{};
        fv.inner4 = make_u32div((uint32_t)(cs[nd - 1] / V));
        fv.inner_stride = (int)ct[nd - 1];
        for (int d = 0; d < 3; ++d) {
            const int src = nd - 2 - d;  // outer dims, innermost of them first
            fv.ext[d] = make_u32div((uint32_t)(src >= 0 ? cs[src] : 1));
            fv.stride[d] = src >= 0 ? ct[src] : 0;
            if (src >= 0 && ct[src] % V != 0) src_vec = false;
        }
        const i64 nv = n / V, blocks = fx::ceil_div(nv, 256);
        if (src_vec) materialize_vec_kernel<T, true><<<dim3((unsigned)blocks), dim3(256), 0, c->stream>>>(in, out, fv, nv);
        else materialize_vec_kernel<T, false><<<dim3((unsigned)blocks), dim3(256), 0, c->stream>>>(in, out, fv, nv);
        FX_LAUNCH_CHECK();
        return FX_OK;
    }
    const i64 blocks = fx::ceil_div(n, 256);
    FX_REQUIRE(blocks <= 0x7fffffff, "fx_materialize: too many elements");
    if (n < (1ll << 31)) {
        CollapsedView cv{};
        cv.nd = nd;
        for (int d = 0; d < nd; ++d) {
            cv.ext[d] = make_u32div((uint32_t)cs[nd - 1 - d]);
            cv.stride[d] = ct[nd - 1 - d];
        }
        materialize_u32_kernel<T><<<dim3((unsigned)blocks), dim3(256), 0, c->stream>>>(in, out, cv, n);
        FX_LAUNCH_CHECK();
        return FX_OK;
    }
    materialize_kernel<T><<<dim3((unsigned)blocks), dim3(256), 0, c->stream>>>(in, out, v, n);
    FX_LAUNCH_CHECK();
    return FX_OK;
}

// ---- synthetic data: counter-based generator (splitmix64 of seed + index), identical for any launch shape ----
__device__ __forceinline__ uint64_t splitmix64(uint64_t x) {
    x += 0x9e3779b97f4a7c15ull;
    x = (x ^ (x >> 30)) * 0xbf58476d1ce4e5b9ull;
    x = (x ^ (x >> 27)) * 0x94d049bb133111ebull;
    return x ^ (x >> 31);
}
// u in [0,1) with 53 (double) or 24 (float) random bits
template <typename T> __device__ __forceinline__ T unit_uniform(uint64_t z);
template <> __device__ __forceinline__ double unit_uniform<double>(uint64_t z) { return (double)(z >> 11) * (1.0 / 9007199254740992.0); }
template <> __device__ __forceinline__ float unit_uniform<float>(uint64_t z) { return (float)(z >> 40) * (1.0f / 16777216.0f); }

template <typename T, bool NORMAL>
__global__ __launch_bounds__(256) void random_fill_kernel(T* __restrict__ out, i64 n, uint64_t seed, T a, T b) {
    const i64 i = (i64)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    if (!NORMAL) {
        out[i] = a + (b - a) * unit_uniform<T>(splitmix64(seed + (uint64_t)i));
    } else {  // Box-Muller; a = mean, b = std
        const double u1 = unit_uniform<double>(splitmix64(seed + 2 * (uint64_t)i));
        const double u2 = unit_uniform<double>(splitmix64(seed + 2 * (uint64_t)i + 1));
        const double r = sqrt(-2.0 * log(1.0 - u1));
        out[i] = (T)((double)a + (double)b * r * cos(6.283185307179586 * u2));
    }
}

template <typename T, bool NORMAL>
int random_fill(fx_ctx* c, T* out, i64 n, uint64_t seed, T a, T b) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(n >= 0, "fx_fill_random: negative element count");
    if (n == 0) return FX_OK;
    FX_REQUIRE(out != nullptr, "fx_fill_random: null pointer");
    const i64 blocks = fx::ceil_div(n, 256);
    FX_REQUIRE(blocks <= 0x7fffffff, "fx_fill_random: too many elements");
    random_fill_kernel<T, NORMAL><<<dim3((unsigned)blocks), dim3(256), 0, c->stream>>>(out, n, seed, a, b);
    FX_LAUNCH_CHECK();
    return FX_OK;
}

// ---- inverted dropout: nn/layers/dropout.rs:56-136 draws one f64 uniform per element, keeps it when u < 1 - p and
// writes mask = 1/(1-p) (cast to T) or 0, then multiplies.  The reference's generator is unseeded; here element i
// takes the 53-bit uniform of splitmix64(seed + i), so a mask can be rebuilt on the host.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void dropout_kernel(const T* __restrict__ x, T* __restrict__ mask, T* __restrict__ y, i64 n,
                                                      uint64_t seed, double keep, T scale) {
    constexpr int V = VEC ? 16 / (int)sizeof(T) : 1;
    typedef T vec_t __attribute__((ext_vector_type(V)));
    const i64 i = ((i64)blockIdx.x * 256 + threadIdx.x) * V;
    if (i >= n) return;
    const vec_t v = *reinterpret_cast<const vec_t*>(x + i);
    vec_t m, r;
#pragma unroll
    for (int u = 0; u < V; ++u) {
        m[u] = unit_uniform<double>(splitmix64(seed + (uint64_t)(i + u))) < keep ? scale : T(0);
        r[u] = v[u] * m[u];
    }
    *reinterpret_cast<vec_t*>(mask + i) = m;
    *reinterpret_cast<vec_t*>(y + i) = r;
}

template <typename T>
int dropout(fx_ctx* c, const T* x, T* mask, T* y, i64 n, double p, uint64_t seed) {
    FX_CHECK_CTX(c);
    FX_REQUIRE(n >= 0, "fx_dropout: negative element count");
    FX_REQUIRE(p >= 0.0 && p < 1.0, "fx_dropout: p must be in [0, 1)");
    if (n == 0) return FX_OK;
    FX_REQUIRE(x && mask && y, "fx_dropout: null pointer");
    constexpr int V = 16 / (int)sizeof(T);
    const bool vec = n % V == 0 && fx::aligned16(x) && fx::aligned16(mask) && fx::aligned16(y);
    const i64 blocks = fx::ceil_div(vec ? n / V : n, 256);
    FX_REQUIRE(blocks <= 0x7fffffff, "fx_dropout: too many elements");
    const double keep = 1.0 - p;
    const T scale = (T)(1.0 / keep);
    if (vec) dropout_kernel<T, true><<<dim3((unsigned)blocks), dim3(256), 0, c->stream>>>(x, mask, y, n, seed, keep, scale);
    else dropout_kernel<T, false><<<dim3((unsigned)blocks), dim3(256), 0, c->stream>>>(x, mask, y, n, seed, keep, scale);
    FX_LAUNCH_CHECK();
    return FX_OK;
}

}  // namespace

#define FX_DEFINE_EW(T, S)                                                                                             \
    extern "C" int fx_dropout_##S(fx_ctx* c, const T* x, T* mask, T* y, int64_t n, double p, uint64_t seed) {          \
        return dropout<T>(c, x, mask, y, n, p, seed);                                                                  \
    }                                                                                                                  \
    extern "C" int fx_fill_uniform_##S(fx_ctx* c, T* out, int64_t n, uint64_t seed, T lo, T hi) {                      \
        return random_fill<T, false>(c, out, n, seed, lo, hi);                                                         \
    }                                                                                                                  \
    extern "C" int fx_fill_normal_##S(fx_ctx* c, T* out, int64_t n, uint64_t seed, T mean, T std) {                    \
        return random_fill<T, true>(c, out, n, seed, mean, std);                                                       \
    }                                                                                                                  \
    extern "C" int fx_fill_##S(fx_ctx* c, T* out, T v, int64_t n) {                                                    \
        return launch_ew<T, 0>(c, (const T*)nullptr, (const T*)nullptr, out, n, FillF<T>{v}, "fx_fill");               \
    }                                                                                                                  \
    extern "C" int fx_materialize_##S(fx_ctx* c, const T* in, T* out, const int64_t* sh, const int64_t* st, int nd,    \
                                      int64_t n) {                                                                     \
        return materialize<T>(c, in, out, sh, st, nd, n);                                                              \
    }                                                                                                                  \
    extern "C" int fx_binary_##S(fx_ctx* c, int op, const T* a, const T* b, T* o, int64_t n) {                         \
        return binary_dispatch<T>(c, op, a, b, o, n);                                                                  \
    }                                                                                                                  \
    extern "C" int fx_add_##S(fx_ctx* c, const T* a, const T* b, T* o, int64_t n) { return binary_dispatch<T>(c, FX_ADD, a, b, o, n); } \
    extern "C" int fx_sub_##S(fx_ctx* c, const T* a, const T* b, T* o, int64_t n) { return binary_dispatch<T>(c, FX_SUB, a, b, o, n); } \
    extern "C" int fx_mul_##S(fx_ctx* c, const T* a, const T* b, T* o, int64_t n) { return binary_dispatch<T>(c, FX_MUL, a, b, o, n); } \
    extern "C" int fx_div_##S(fx_ctx* c, const T* a, const T* b, T* o, int64_t n) { return binary_dispatch<T>(c, FX_DIV, a, b, o, n); } \
    extern "C" int fx_equal_##S(fx_ctx* c, const T* a, const T* b, T* o, int64_t n) { return binary_dispatch<T>(c, FX_EQUAL, a, b, o, n); } \
    extern "C" int fx_scalar_##S(fx_ctx* c, int op, const T* a, T s, T* o, int64_t n) {                                \
        return scalar_dispatch<T>(c, op, a, s, o, n);                                                                  \
    }                                                                                                                  \
    extern "C" int fx_add_scalar_##S(fx_ctx* c, const T* a, T s, T* o, int64_t n) { return scalar_dispatch<T>(c, FX_ADD_SCALAR, a, s, o, n); } \
    extern "C" int fx_sub_scalar_##S(fx_ctx* c, const T* a, T s, T* o, int64_t n) { return scalar_dispatch<T>(c, FX_SUB_SCALAR, a, s, o, n); } \
    extern "C" int fx_mul_scalar_##S(fx_ctx* c, const T* a, T s, T* o, int64_t n) { return scalar_dispatch<T>(c, FX_MUL_SCALAR, a, s, o, n); } \
    extern "C" int fx_div_scalar_##S(fx_ctx* c, const T* a, T s, T* o, int64_t n) { return scalar_dispatch<T>(c, FX_DIV_SCALAR, a, s, o, n); } \
    extern "C" int fx_greater_scalar_##S(fx_ctx* c, const T* a, T s, T* o, int64_t n) { return scalar_dispatch<T>(c, FX_GREATER_SCALAR, a, s, o, n); } \
    extern "C" int fx_greater_equal_scalar_##S(fx_ctx* c, const T* a, T s, T* o, int64_t n) { return scalar_dispatch<T>(c, FX_GREATER_EQUAL_SCALAR, a, s, o, n); } \
    extern "C" int fx_less_equal_scalar_##S(fx_ctx* c, const T* a, T s, T* o, int64_t n) { return scalar_dispatch<T>(c, FX_LESS_EQUAL_SCALAR, a, s, o, n); } \
    extern "C" int fx_unary_##S(fx_ctx* c, int op, const T* a, T* o, int64_t n) { return unary_dispatch<T>(c, op, a, o, n); } \
    extern "C" int fx_neg_##S(fx_ctx* c, const T* a, T* o, int64_t n) { return unary_dispatch<T>(c, FX_NEG, a, o, n); } \
    extern "C" int fx_sqrt_##S(fx_ctx* c, const T* a, T* o, int64_t n) { return unary_dispatch<T>(c, FX_SQRT, a, o, n); } \
    extern "C" int fx_exp_##S(fx_ctx* c, const T* a, T* o, int64_t n) { return unary_dispatch<T>(c, FX_EXP, a, o, n); } \
    extern "C" int fx_log_##S(fx_ctx* c, const T* a, T* o, int64_t n) { return unary_dispatch<T>(c, FX_LOG, a, o, n); } \
    extern "C" int fx_relu_##S(fx_ctx* c, const T* a, T* o, int64_t n) { return unary_dispatch<T>(c, FX_RELU, a, o, n); } \
    extern "C" int fx_sigmoid_##S(fx_ctx* c, const T* a, T* o, int64_t n) { return unary_dispatch<T>(c, FX_SIGMOID, a, o, n); } \
    extern "C" int fx_tanh_##S(fx_ctx* c, const T* a, T* o, int64_t n) { return unary_dispatch<T>(c, FX_TANH, a, o, n); } \
    extern "C" int fx_clamp_##S(fx_ctx* c, const T* a, T lo, T hi, T* o, int64_t n) {                                  \
        return launch_ew<T, 1>(c, a, (const T*)nullptr, o, n, ClampF<T>{lo, hi}, "fx_clamp");                          \
    }                                                                                                                  \
    extern "C" int fx_in_range_##S(fx_ctx* c, const T* a, T lo, T hi, T* o, int64_t n) {                               \
        return launch_ew<T, 1>(c, a, (const T*)nullptr, o, n, InRangeF<T>{lo, hi}, "fx_in_range");                     \
    }                                                                                                                  \
    extern "C" int fx_relu_bwd_##S(fx_ctx* c, const T* g, const T* x, T* o, int64_t n) {                               \
        return launch_ew<T, 2>(c, g, x, o, n, ReluBwdF<T>{}, "fx_relu_bwd");                                           \
    }                                                                                                                  \
    extern "C" int fx_sigmoid_bwd_##S(fx_ctx* c, const T* g, const T* s, T* o, int64_t n, int literal) {               \
        return literal ? launch_ew<T, 2>(c, g, s, o, n, SigmoidBwdF<T, 1>{}, "fx_sigmoid_bwd")                         \
                       : launch_ew<T, 2>(c, g, s, o, n, SigmoidBwdF<T, 0>{}, "fx_sigmoid_bwd");                        \
    }                                                                                                                  \
    extern "C" int fx_tanh_bwd_##S(fx_ctx* c, const T* g, const T* t, T* o, int64_t n) {                               \
        return launch_ew<T, 2>(c, g, t, o, n, TanhBwdF<T>{}, "fx_tanh_bwd");                                           \
    }

FX_DEFINE_EW(float, f32)
FX_DEFINE_EW(double, f64)

// Device-to-device copy of a small block as a streaming kernel on the context's stream.  A hipMemcpyAsync D2D of a few KB
// to a few MB occupies the stream about twice as long as this kernel (a training step of the op-by-op engines issues dozens
// of such clones).  4-byte granularity; returns FX_ERR_UNSUPPORTED for anything else so the caller can fall back.
namespace fx {
int copy_kernel(fx_ctx* c, void* dst, const void* src, i64 bytes) {
    if ((bytes & 3) != 0 || (reinterpret_cast<uintptr_t>(dst) & 3u) != 0 || (reinterpret_cast<uintptr_t>(src) & 3u) != 0)
        return FX_ERR_UNSUPPORTED;
    return launch_ew<float, 1>(c, static_cast<const float*>(src), (const float*)nullptr, static_cast<float*>(dst), bytes / 4,
                               CopyF<float>{}, "fx_d2d");
}
}  // namespace fx
