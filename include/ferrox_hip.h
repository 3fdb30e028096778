/*
 * ferrox_hip.h -- C ABI of libferrox_hip.so, the MI355X (gfx950) backend for Ferrox's training hot path.
 *
 * This is the boundary a `HipStorage<T>: StorageBackend<T>` implementation binds through FFI.  It replaces,
 * one for one, what the reference reaches through cudarc:
 *   - CudaContextManager  (src/backend/cuda/context.rs:30-175)   -> fx_init / fx_destroy / fx_sync / copies
 *   - CudaMemoryPool      (src/backend/memory/cuda.rs:55-134)    -> fx_alloc / fx_free / fx_pool_*
 *   - KernelManager::launch_* (src/backend/cuda/kernels.rs:435-1918) -> the fx_<op>_{f32,f64} kernel entry points
 *
 * Conventions
 *   - Every function returns an int status: FX_OK (0) or an FX_ERR_* code; the message of the last failure on
 *     the calling thread is available from fx_last_error().
 *   - All tensor pointers are DEVICE pointers unless the parameter is named host_*.  Sizes and counts are
 *     int64_t ELEMENTS unless named *_bytes.  Shapes are row-major (C order), exactly as Ferrox stores them.
 *   - Every kernel is enqueued on the context's single compute stream and returns without waiting; call
 *     fx_sync() (or a device-to-host copy, which waits) before reading results on the host.
 *   - Memory handed out by the pool is NOT zeroed on reuse (as in the reference, context.rs:72-73); every
 *     kernel here fully defines its output.
 *   - A context may be used from several host threads; allocator calls are serialised internally and launches
 *     are serialised per context.  Every entry point makes the context's device current on the calling thread.
 *   - dtype suffixes: _f32 = float, _f64 = double.  The reference names its kernels `op` / `op_f64`
 *     (src/backend/cuda/kernels.rs:283-292).
 */
#ifndef FERROX_HIP_H
#define FERROX_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FX_OK 0
#define FX_ERR_INVALID 1     /* bad argument / shape mismatch */
#define FX_ERR_HIP 2         /* a HIP runtime call failed */
#define FX_ERR_OOM 3         /* device allocation failed */
#define FX_ERR_UNSUPPORTED 4 /* valid request this build does not serve */

#define FX_F32 0
#define FX_F64 1

typedef struct fx_ctx fx_ctx;

/* ---- allocator configuration: PoolConfig / BucketConfig, src/backend/memory/mod.rs:15-82 ---------------- */
#define FX_MAX_BUCKETS 8
typedef struct fx_bucket_config {
    int64_t min_elems;              /* inclusive */
    int64_t max_elems;              /* inclusive; INT64_MAX for "no limit" */
    int64_t max_blocks;             /* max_allocations */
    int64_t to_evict;               /* blocks dropped at once when the bucket is full (LRU) */
    int64_t eviction_threshold_ms;  /* >= 0: evict blocks older than this instead of LRU; < 0: none */
} fx_bucket_config;

typedef struct fx_pool_config {
    int32_t n_buckets;   /* 0 = the library default: the four size classes of PoolConfig::default() (mod.rs:50-82:
                            <=1024, <=262144, <=16777216, larger) holding 4096/1024/256/16 blocks instead of the
                            reference's 500/50/10/2, which were sized for a 4-8 GB card */
    int32_t literal_ids; /* 1 = keep the reference's id bookkeeping (a reused block keeps its old id, so its second
                            release is dropped, cuda.rs:61-62,76-87); 0 = a reused block is re-registered (default) */
    int32_t best_fit;    /* 0 = the reference's policy: only the most recently returned block of the bucket is tried
                            (cuda.rs:79-92), a too-small one is an underflow miss; 1 = the smallest pooled block of the
                            bucket that is large enough is taken (most recent among equals), which removes most
                            underflow misses.  fx_init(cfg = NULL) uses best_fit = 1, literal_ids = 0. */
    int32_t reserved;
    fx_bucket_config buckets[FX_MAX_BUCKETS];
} fx_pool_config;

/* PoolStats, src/backend/memory/mod.rs:195-202, plus what print_stats derives (cuda.rs:138-185) */
typedef struct fx_pool_stats {
    int64_t total_allocations;
    int64_t active_allocations;
    int64_t pool_hits;
    int64_t pool_misses;
    int64_t underflow_misses;
    int64_t allocation_counter; /* CudaMemoryPool::allocation_counter */
    int64_t active_table_len;   /* active_allocations.len() */
    int64_t device_allocs;      /* hipMalloc calls made for this pool */
    int64_t device_frees;       /* hipFree calls made for this pool */
    int64_t bytes_in_use;       /* bytes currently handed out */
    int64_t bytes_pooled;       /* bytes cached in buckets */
    int64_t peak_bytes;         /* high-water mark of in_use + pooled */
} fx_pool_stats;

/* BucketStats, src/backend/memory/mod.rs:204-222 */
typedef struct fx_bucket_stats {
    int64_t pooled_blocks;
    int64_t total_allocations;
    int64_t total_evictions;
    int64_t av_allocations;
    int64_t max_allocations;
} fx_bucket_stats;

/* ---- runtime: CudaContextManager::{from_device_id, synchronize, name}, context.rs:35-59, 152-172 -------- */
int fx_init(int device, const fx_pool_config* cfg_or_null, fx_ctx** out);
int fx_destroy(fx_ctx* ctx);
int fx_sync(fx_ctx* ctx);
int fx_device_name(fx_ctx* ctx, char* buf, int64_t buf_len);
const char* fx_last_error(void);
/* The compute stream as a hipStream_t (for callers that enqueue their own work behind the library's). */
void* fx_stream(fx_ctx* ctx);

/* Stream timing for benchmarks (the reference times with cudaEvent pairs, kernels/benchmark.cu:575-603):
 * fx_timer_start records an event on the compute stream, fx_timer_stop records a second one, waits for it and
 * returns the elapsed milliseconds between the two. */
int fx_timer_start(fx_ctx* ctx);
int fx_timer_stop(fx_ctx* ctx, float* elapsed_ms);

/* ---- allocator: CudaMemoryPool::{allocate, deallocate, cleanup, reset, stats}, memory/cuda.rs:55-134 ----- */
/* n_elems == 0 -> FX_ERR_INVALID "Cannot allocate zero-sized CUDA memory" (cuda.rs:57-59).
 * *granted_elems may exceed n_elems on a pool hit (the reference truncates on read-back, context.rs:410-426). */
int fx_alloc(fx_ctx* ctx, int dtype, int64_t n_elems, void** ptr, int64_t* granted_elems, uint64_t* alloc_id);
/* A pointer the pool does not own, or one that was already released, is an error (FX_ERR_INVALID). */
int fx_free(fx_ctx* ctx, int dtype, void* ptr, uint64_t alloc_id);
int fx_pool_cleanup(fx_ctx* ctx, int dtype);
int fx_pool_reset(fx_ctx* ctx, int dtype);
int fx_pool_stats_get(fx_ctx* ctx, int dtype, fx_pool_stats* out);
int fx_pool_bucket_stats_get(fx_ctx* ctx, int dtype, int bucket, fx_bucket_stats* out);

/* ---- copies: host_to_device / device_to_host / device_to_device, context.rs:81-150 (synchronous) -------- */
int fx_h2d(fx_ctx* ctx, void* dst_dev, const void* host_src, int64_t bytes);
int fx_d2h(fx_ctx* ctx, void* host_dst, const void* src_dev, int64_t bytes);
int fx_d2d(fx_ctx* ctx, void* dst_dev, const void* src_dev, int64_t bytes);

/* ---- workspace queries ---------------------------------------------------------------------------------- */
#define FX_CONV_FWD 0
#define FX_CONV_DGRAD 1
#define FX_CONV_WGRAD 2
/* Bytes of scratch fx_conv2d_* needs for this shape.  Passing workspace == NULL to the conv entry points makes
 * the library use (and grow) its own per-context scratch instead. */
int64_t fx_conv2d_workspace_bytes(int kind, int dtype, int mode, int64_t B, int64_t Cin, int64_t H, int64_t W,
                                  int64_t Cout, int64_t kh, int64_t kw, int64_t sh, int64_t sw, int64_t ph, int64_t pw);

/* Tile-shape timing of the 3x3 f32 convolutions.  fx_conv2d_fwd_f32 (and its bias variant) and fx_conv2d_dgrad_f32 pick
 * the tile shape of their LDS-patch kernel by measurement: the FIRST call for a layer (filter / map / channel sizes,
 * stride, padding, epilogue) and batch size class floor(log2(B)) launches every near-tied shape a few times on the
 * caller's own tensors and waits for the stream once per shape (about 4 launches per shape, up to 11 shapes), then
 * remembers the winner in the context; every later call is one asynchronous launch.  All shapes write the same complete
 * output with the same bits, so only latency differs.  The output must not overlap an operand (then nothing is timed and
 * the modelled shape is used).  FX_CONV_TUNE=0 in the environment switches the timing off.  fx_conv2d_tune_f32 pays that
 * cost up front for a layer (kind FX_CONV_FWD or FX_CONV_DGRAD; FX_CONV_WGRAD is accepted and has nothing to time), on
 * temporary zero-filled tensors it allocates and frees itself; it synchronises the stream.  with_bias / act select the
 * epilogue of fx_conv2d_fwd_bias_act (both 0 for plain fx_conv2d_fwd).  No counterpart in the reference (its kernels have
 * one fixed launch geometry, src/backend/cuda/ops.rs:57-118). */
int fx_conv2d_tune_f32(fx_ctx* ctx, int kind, int64_t B, int64_t Cin, int64_t H, int64_t W, int64_t Cout, int64_t kh,
                       int64_t kw, int64_t sh, int64_t sw, int64_t ph, int64_t pw, int with_bias, int act);

/* Binary / scalar / unary op selectors for the generic entry points (also exported one by one below). */
enum fx_binary_op { FX_ADD = 0, FX_SUB = 1, FX_MUL = 2, FX_DIV = 3, FX_EQUAL = 4, FX_GREATER = 5, FX_GREATER_EQUAL = 6,
                    FX_LESS = 7, FX_LESS_EQUAL = 8, FX_MIN = 9, FX_MAX = 10, FX_POW = 11 };
enum fx_unary_op { FX_NEG = 0, FX_SQRT = 1, FX_EXP = 2, FX_LOG = 3, FX_RELU = 4, FX_SIGMOID = 5, FX_TANH = 6, FX_ABS = 7,
                   FX_RECIPROCAL = 8, FX_SIGN = 9, FX_LOGICAL_NOT = 10 };
enum fx_scalar_op { FX_ADD_SCALAR = 0, FX_SUB_SCALAR = 1, FX_MUL_SCALAR = 2, FX_DIV_SCALAR = 3, FX_GREATER_SCALAR = 4,
                    FX_GREATER_EQUAL_SCALAR = 5, FX_LESS_EQUAL_SCALAR = 6, FX_LESS_SCALAR = 7, FX_POW_SCALAR = 8 };

#define FX_DECLARE_KERNELS(T, S)                                                                                       \
    /* launch_fill, kernels.rs:435-448 */                                                                              \
    int fx_fill_##S(fx_ctx* ctx, T* out, T value, int64_t n);                                                          \
    /* launch_fill_random, kernels.rs:450-467 (kernels/fill.cu:7-21 hashes seed+idx with xorshift32 into U(-1,1)).     \
       Here: splitmix64(seed + i) -> lo + (hi-lo)*u, u in [0,1) with 24/53 random bits; reproducible on the host        \
       with integer arithmetic.  The normal variant applies Box-Muller to hashes 2i and 2i+1. */                       \
    int fx_fill_uniform_##S(fx_ctx* ctx, T* out, int64_t n, uint64_t seed, T lo, T hi);                                \
    int fx_fill_normal_##S(fx_ctx* ctx, T* out, int64_t n, uint64_t seed, T mean, T std);                              \
    /* launch_materialize, kernels.rs:802-830 / CudaOps::materialize, ops.rs:175-214.  shape and strides (in          \
       elements, 0 on broadcast dims) are HOST arrays, ndim <= 8. */                                                   \
    int fx_materialize_##S(fx_ctx* ctx, const T* in, T* out, const int64_t* host_shape, const int64_t* host_strides,   \
                           int ndim, int64_t n);                                                                       \
    /* launch_add/sub/mul/div/min/max + comparisons, kernels.rs:469-585, 940-1075.  Same-shape operands only           \
       (cpu.rs:629-690).  Comparisons write 1.0 / 0.0.  a/0 follows IEEE like the CPU backend. */                      \
    int fx_binary_##S(fx_ctx* ctx, int op, const T* a, const T* b, T* out, int64_t n);                                 \
    int fx_add_##S(fx_ctx* ctx, const T* a, const T* b, T* out, int64_t n);                                            \
    int fx_sub_##S(fx_ctx* ctx, const T* a, const T* b, T* out, int64_t n);                                            \
    int fx_mul_##S(fx_ctx* ctx, const T* a, const T* b, T* out, int64_t n);                                            \
    int fx_div_##S(fx_ctx* ctx, const T* a, const T* b, T* out, int64_t n);                                            \
    int fx_equal_##S(fx_ctx* ctx, const T* a, const T* b, T* out, int64_t n);                                          \
    /* scalar ops, CudaOps::{add,sub,mul,div}_scalar ops.rs:435-464 (the reference fills a full-size temp first;       \
       here the scalar is a kernel argument) and launch_*_scalar, kernels.rs:954-1010 */                               \
    int fx_scalar_##S(fx_ctx* ctx, int op, const T* a, T s, T* out, int64_t n);                                        \
    int fx_add_scalar_##S(fx_ctx* ctx, const T* a, T s, T* out, int64_t n);                                            \
    int fx_sub_scalar_##S(fx_ctx* ctx, const T* a, T s, T* out, int64_t n);                                            \
    int fx_mul_scalar_##S(fx_ctx* ctx, const T* a, T s, T* out, int64_t n);                                            \
    int fx_div_scalar_##S(fx_ctx* ctx, const T* a, T s, T* out, int64_t n);                                            \
    int fx_greater_scalar_##S(fx_ctx* ctx, const T* a, T s, T* out, int64_t n);                                        \
    int fx_greater_equal_scalar_##S(fx_ctx* ctx, const T* a, T s, T* out, int64_t n);                                  \
    int fx_less_equal_scalar_##S(fx_ctx* ctx, const T* a, T s, T* out, int64_t n);                                     \
    /* unary ops, kernels.rs:587-740 (abs, sqrt, exp, log, negate, sigmoid, tanh, relu).  tanh saturates to +-1        \
       beyond |x| > 20 like cpu.rs:1112-1119. */                                                                       \
    int fx_unary_##S(fx_ctx* ctx, int op, const T* a, T* out, int64_t n);                                              \
    int fx_neg_##S(fx_ctx* ctx, const T* a, T* out, int64_t n);                                                        \
    int fx_sqrt_##S(fx_ctx* ctx, const T* a, T* out, int64_t n);                                                       \
    int fx_exp_##S(fx_ctx* ctx, const T* a, T* out, int64_t n);                                                        \
    int fx_log_##S(fx_ctx* ctx, const T* a, T* out, int64_t n);                                                        \
    int fx_relu_##S(fx_ctx* ctx, const T* a, T* out, int64_t n);                                                       \
    int fx_sigmoid_##S(fx_ctx* ctx, const T* a, T* out, int64_t n);                                                    \
    int fx_tanh_##S(fx_ctx* ctx, const T* a, T* out, int64_t n);                                                       \
    /* launch_clamp, kernels.rs:894-917 / cpu.rs:792-805 */                                                            \
    int fx_clamp_##S(fx_ctx* ctx, const T* a, T lo, T hi, T* out, int64_t n);                                          \
    /* in_range, cpu.rs:933-947: 1 where lo <= a <= hi, else 0.  (min/max/greater/less... of two tensors, sign,        \
       logical_not, powf and power_scalar -- cpu.rs:692-740, 815-965, 1152-1182 -- go through the fx_binary /          \
       fx_unary / fx_scalar selectors.) */                                                                             \
    int fx_in_range_##S(fx_ctx* ctx, const T* a, T lo, T hi, T* out, int64_t n);                                       \
    /* Fused activation gradients.  The reference has no backward kernels: ReLU::gradient, Sigmoid::gradient and       \
       Tanh::gradient (src/ops/unary.rs:358-375, 254-276, 306-328) compose 2-4 storage ops.  These produce the         \
       same values in one pass: relu: g*(x>0); tanh: g*(-(t*t-1)); sigmoid: literal=1 -> g*(s*(s-1)) (the              \
       reference's sign), literal=0 -> g*(s*(1-s)). */                                                                 \
    int fx_relu_bwd_##S(fx_ctx* ctx, const T* g, const T* x, T* out, int64_t n);                                       \
    int fx_sigmoid_bwd_##S(fx_ctx* ctx, const T* g, const T* s, T* out, int64_t n, int literal);                       \
    int fx_tanh_bwd_##S(fx_ctx* ctx, const T* g, const T* t, T* out, int64_t n);                                       \
    /* launch_softmax_batched, kernels.rs:683-711 / cpu.rs:1037-1068: softmax over `axis` of [outer, axis, inner] */   \
    int fx_softmax_axis_##S(fx_ctx* ctx, const T* in, T* out, int64_t outer, int64_t axis, int64_t inner);             \
    /* launch_sum_axes / launch_max_axes / launch_*_all, kernels.rs:742-800; CudaOps::reduce_axes ops.rs:2171-2284;    \
       cpu.rs:1183-1238.  Reduces the middle dimension of a contiguous [outer, axis, inner] view into                  \
       [outer, inner]; "all" = (1, n, 1).  mean multiplies the sum by T(1/axis) (cpu.rs:1217-1220).  max starts        \
       from the lowest finite T and takes strictly greater values (cpu.rs:1231-1234); idx_out (may be NULL)            \
       receives the FIRST index along the axis that attains the maximum, as int64. */                                  \
    int fx_reduce_sum_##S(fx_ctx* ctx, const T* in, T* out, int64_t outer, int64_t axis, int64_t inner);               \
    int fx_reduce_mean_##S(fx_ctx* ctx, const T* in, T* out, int64_t outer, int64_t axis, int64_t inner);              \
    int fx_reduce_max_##S(fx_ctx* ctx, const T* in, T* out, int64_t* idx_out, int64_t outer, int64_t axis,             \
                          int64_t inner);                                                                              \
    /* min_reduce, cpu.rs:1240-1252: starts from the highest finite T, takes strictly smaller values; idx_out as above. */ \
    int fx_reduce_min_##S(fx_ctx* ctx, const T* in, T* out, int64_t* idx_out, int64_t outer, int64_t axis,             \
                          int64_t inner);                                                                              \
    /* reduce_prod_all / reduce_prod_axes, kernels/reduction.cu:232-301, 348-360: product along the axis, from 1. */    \
    int fx_reduce_prod_##S(fx_ctx* ctx, const T* in, T* out, int64_t outer, int64_t axis, int64_t inner);              \
    /* launch_matmul, kernels.rs:919-938 / cpu.rs:967-1002: C[M,N] = op(A) . op(B).  trans_a: A is stored [K,M];       \
       trans_b: B is stored [N,K]  (lets MatMul::gradient, src/ops/matrix.rs:30-55, skip materialised transposes). */  \
    int fx_gemm_##S(fx_ctx* ctx, int trans_a, int trans_b, int64_t M, int64_t N, int64_t K, const T* A, const T* B,    \
                    T* C);                                                                                             \
    /* im2col / col2im, src/backend/storage/extensions/convolutions.rs:10-75, 79-153.                                  \
       col is [C*kh*kw, B*oh*ow] row-major.  col2im layout 0 reads it that way; layout 1 reads the buffer with the     \
       reference's batch-major flat index (convolutions.rs:122-127).  The sum for each pixel runs over (ky, kx)        \
       ascending, the reference's loop order, so results are bit-identical to the CPU. */                              \
    int fx_im2col_##S(fx_ctx* ctx, const T* x, T* col, int64_t B, int64_t C, int64_t H, int64_t W, int64_t kh,         \
                      int64_t kw, int64_t sh, int64_t sw, int64_t ph, int64_t pw);                                     \
    int fx_col2im_##S(fx_ctx* ctx, const T* col, T* out, int64_t B, int64_t C, int64_t H, int64_t W, int64_t kh,       \
                      int64_t kw, int64_t sh, int64_t sw, int64_t ph, int64_t pw, int layout);                         \
    /* launch_conv2d_forward / launch_deconv2d / launch_cross_correlation2d, kernels.rs:1213-1256, 1340-1384,          \
       1386-1430; CPU path convolutions.rs:218-338.  NCHW.  oh = (H+2ph-kh)/sh+1.                                      \
       fwd:   y[B,Cout,oh,ow]   = conv(x[B,Cin,H,W], w[Cout,Cin,kh,kw])                                                \
       dgrad: dx[B,Cin,H,W]     from g[B,Cout,oh,ow], w                                                                \
       wgrad: dw[Cout,Cin,kh,kw] from x, g                                                                             \
       mode 0 = the mathematical gradient (what the reference's CUDA kernels compute); mode 1 = the CPU backend's      \
       literal arithmetic (flat reinterpretation of g as [Cout, B*L] and batch-major col2im), which equals mode 0       \
       only for batch 1. */                                                                                            \
    int fx_conv2d_fwd_##S(fx_ctx* ctx, const T* x, const T* w, T* y, int64_t B, int64_t Cin, int64_t H, int64_t W,     \
                          int64_t Cout, int64_t kh, int64_t kw, int64_t sh, int64_t sw, int64_t ph, int64_t pw,        \
                          void* workspace, int64_t ws_bytes);                                                          \
    int fx_conv2d_dgrad_##S(fx_ctx* ctx, const T* g, const T* w, T* dx, int64_t B, int64_t Cin, int64_t H, int64_t W,  \
                            int64_t Cout, int64_t kh, int64_t kw, int64_t sh, int64_t sw, int64_t ph, int64_t pw,      \
                            int mode, void* workspace, int64_t ws_bytes);                                              \
    int fx_conv2d_wgrad_##S(fx_ctx* ctx, const T* x, const T* g, T* dw, int64_t B, int64_t Cin, int64_t H, int64_t W,  \
                            int64_t Cout, int64_t kh, int64_t kw, int64_t sh, int64_t sw, int64_t ph, int64_t pw,      \
                            int mode, void* workspace, int64_t ws_bytes);                                              \
    /* maxpool2d / avgpool2d and their gradients max_unpool2d / avg_unpool2d, storage/mod.rs:328-420 ->                \
       extensions/pooling.rs:154-229, 339-418 (launch_maxpool2d... kernels.rs; kernels/convolutions.cu:671-1222).      \
       NCHW, out is [N, C, (H+2ph-kh)/sh+1, (W+2pw-kw)/sw+1]; the reference's square window / single stride is         \
       kh == kw, sh == sw; the 1-D calls ([N, C, L]) are H = 1, kh = 1, sh = 1, ph = 0.  Bit-identical to the CPU      \
       loops: max from the lowest finite T with strict >, avg over the in-bounds count, max gradient where             \
       |in - pooled| < 1e-8, avg gradient scaled by T(1.0f / float(kh*kw)). */                                         \
    int fx_maxpool2d_##S(fx_ctx* ctx, const T* in, T* out, int64_t N, int64_t C, int64_t H, int64_t W, int64_t kh,     \
                         int64_t kw, int64_t sh, int64_t sw, int64_t ph, int64_t pw);                                  \
    int fx_avgpool2d_##S(fx_ctx* ctx, const T* in, T* out, int64_t N, int64_t C, int64_t H, int64_t W, int64_t kh,     \
                         int64_t kw, int64_t sh, int64_t sw, int64_t ph, int64_t pw);                                  \
    int fx_max_unpool2d_##S(fx_ctx* ctx, const T* grad_out, const T* in, const T* pooled, T* grad_in, int64_t N,       \
                            int64_t C, int64_t H, int64_t W, int64_t kh, int64_t kw, int64_t sh, int64_t sw,           \
                            int64_t ph, int64_t pw);                                                                   \
    int fx_avg_unpool2d_##S(fx_ctx* ctx, const T* grad_out, T* grad_in, int64_t N, int64_t C, int64_t H, int64_t W,    \
                            int64_t kh, int64_t kw, int64_t sh, int64_t sw, int64_t ph, int64_t pw);                   \
    /* ---- fused sequences (optional: every one equals a chain of the entry points above) ----                        \
       Bias add, in place, on y viewed as [outer, C, inner] (conv: outer = B, inner = oh*ow; linear: outer = B,        \
       inner = 1), act 0 = none, 1 = ReLU.  Replaces Reshape + BroadcastTo + Add (+ ReLU) of                           \
       src/nn/layers/utils.rs:6-42, conv2d.rs:203-213, linear.rs:262-279; same values bit for bit. */                  \
    int fx_bias_act_##S(fx_ctx* ctx, T* y, const T* bias, int64_t outer, int64_t C, int64_t inner, int act);           \
    /* The same bias add (+ ReLU) carried in the store of the producing kernel: fx_conv2d_fwd / fx_gemm followed by     \
       fx_bias_act, in one pass over the output (bias per output channel for the conv, per column of C for the GEMM);   \
       bit-identical to the two-call sequence. */                                                                      \
    int fx_conv2d_fwd_bias_act_##S(fx_ctx* ctx, const T* x, const T* w, const T* bias, T* y, int64_t B, int64_t Cin,   \
                                   int64_t H, int64_t W, int64_t Cout, int64_t kh, int64_t kw, int64_t sh, int64_t sw, \
                                   int64_t ph, int64_t pw, int act, void* workspace, int64_t ws_bytes);                \
    int fx_gemm_bias_act_##S(fx_ctx* ctx, int trans_a, int trans_b, int64_t M, int64_t N, int64_t K, const T* A,       \
                             const T* B, const T* bias, T* C, int act);                                                \
    /* Backward of a convolution whose output went through a ReLU (Conv2dOp::gradient, src/ops/batched.rs:194-217,     \
       after ReLU::gradient, src/ops/unary.rs:358-375, and the bias reduction of src/ops/basic.rs:10-53), from the     \
       UNMASKED upstream gradient g and the layer's activation act = relu(conv(x) + b), both [B,Cout,oh,ow]:           \
         wgrad_relu_bias: dw = fx_conv2d_wgrad(x, g'), db[oc] = sum over (b, pixel) of g'      with g' = g*(act > 0)   \
         dgrad_relu:      dx = fx_conv2d_dgrad(g', w)                                                                   \
       g' is formed while the kernels stage g (the bits of fx_relu_bwd) and is never written: the separate mask +      \
       bias pass and its read-back disappear.  Gradient mode 0 only.  dw and dx have the bits of the two-call          \
       sequences; db is summed in the kernel's own fixed order (equal to fx_bias_grad up to rounding).  Served for     \
       the shapes fx_conv2d_bwd_relu_supported reports (3x3 image layers of at most 3 channels -- f64: maps 32 wide --  \
       and 3x3 stride-2 padding-1 layers over even maps 32 or 64 wide; the weight gradient also over maps 56, 28 and   \
       16 wide); any other call returns FX_ERR_UNSUPPORTED and changes nothing.                                        \
       workspace as for fx_conv2d_wgrad (fx_conv2d_workspace_bytes(FX_CONV_WGRAD, ...) covers it). */                  \
    int fx_conv2d_wgrad_relu_bias_##S(fx_ctx* ctx, const T* x, const T* g, const T* act, T* dw, T* db, int64_t B,      \
                                      int64_t Cin, int64_t H, int64_t W, int64_t Cout, int64_t kh, int64_t kw,         \
                                      int64_t sh, int64_t sw, int64_t ph, int64_t pw, void* workspace,                 \
                                      int64_t ws_bytes);                                                               \
    int fx_conv2d_dgrad_relu_##S(fx_ctx* ctx, const T* g, const T* act, const T* w, T* dx, int64_t B, int64_t Cin,     \
                                 int64_t H, int64_t W, int64_t Cout, int64_t kh, int64_t kw, int64_t sh, int64_t sw,   \
                                 int64_t ph, int64_t pw);                                                              \
    /* Linear's weight and bias gradient in one call (nn/layers/linear.rs:152-308: MatMul::gradient, ops/matrix.rs:    \
       34-55, and reduce_gradient_for_broadcasting, ops/basic.rs:10-53): C[M,N] = A^T . B for A = dY stored [K, M] and \
       B = X stored [K, N] -- fx_gemm(1, 0, ...) up to the order of summation -- and colsum[m] = sum over k of         \
       A[k][m], in a fixed order of its own (equal to fx_bias_grad(A, K, M, 1) up to rounding).  Small and thin        \
       products write the sums from the product's launch; the others run the bias-gradient kernel after it. */         \
    int fx_gemm_tn_colsum_##S(fx_ctx* ctx, int64_t M, int64_t N, int64_t K, const T* A, const T* B, T* C, T* colsum);  \
    /* Linear's backward products in one call (nn/layers/linear.rs:152-308, MatMul::gradient ops/matrix.rs:34-55):     \
       dX[B, in] = dY[B, out] . W[out, in], dW[out, in] = dY^T . X[B, in] and, with db != NULL, db[out] = the column   \
       sums of dY.  dX and dW are fx_gemm(0, 0, ...) and fx_gemm(1, 0, ...) up to the order of summation (a fixed one  \
       per shape), dW and db have the bits of fx_gemm_tn_colsum; two small products share one launch.                  \
       relu_below != 0: X is the output of a ReLU (the layer below ends in one) and dX is the gradient of that ReLU's  \
       input, fx_relu_bwd(dY . W, X) (ReLU::gradient, ops/unary.rs:358-375) -- in the product's store where the        \
       products share a launch. */                                                                                     \
    int fx_linear_bwd_##S(fx_ctx* ctx, int64_t B, int64_t in, int64_t out, const T* dY, const T* W, const T* X, T* dX, \
                          T* dW, T* db, int relu_below);                                                               \
    /* BatchNorm, src/nn/layers/norm.rs:127-336, on x viewed as [outer, C, inner] ([N,C,H,W]: outer = N, inner = H*W;   \
       [N,F]: C = F, inner = 1).  stats: mean[C] and biased variance[C] of every channel in one read of x (the         \
       reference's Mean, Sub, Mul, Mean chain), and, when the pointers are not NULL, the running update                \
       running = running*(1-momentum) + batch*momentum (norm.rs:144-161).  fwd: y = ((x-mean)/sqrt(var+eps))*gamma     \
       + beta, the composed operations in the composed order, bit-identical to them given mean and var (pass the       \
       running statistics for inference, norm.rs:261-290); act 1 applies the ReLU that follows the layer in the        \
       reference's models (activation.rs:47-80) in the same store.  bwd: dgamma[C], dbeta[C] and, unless dx is NULL,   \
       dx; batch_stats 1 = mean/var came from this batch (gradient flows through them), 0 = fixed statistics;          \
       y_act NULL, or the output of the act = 1 forward: dy is then the gradient of that output and counts only       \
       where y_act > 0 (ReLU::gradient, ops/unary.rs:358-375). */                                                      \
    int fx_batchnorm_stats_##S(fx_ctx* ctx, const T* x, T* mean, T* var, T* running_mean, T* running_var,              \
                               double momentum, int64_t outer, int64_t C, int64_t inner);                              \
    int fx_batchnorm_fwd_##S(fx_ctx* ctx, const T* x, const T* mean, const T* var, const T* gamma, const T* beta,      \
                             double eps, T* y, int64_t outer, int64_t C, int64_t inner, int act);                      \
    int fx_batchnorm_bwd_##S(fx_ctx* ctx, const T* dy, const T* x, const T* y_act, const T* mean, const T* var,        \
                             const T* gamma, double eps, T* dx, T* dgamma, T* dbeta, int64_t outer, int64_t C,         \
                             int64_t inner, int batch_stats);                                                          \
    /* Dropout::forward in training, src/nn/layers/dropout.rs:56-136: mask[i] = 1/(1-p) where u_i < 1-p, else 0, and    \
       y = x*mask; u_i is the 53-bit uniform of splitmix64(seed + i) (the reference's generator is unseeded), 0 <= p    \
       < 1.  The gradient is fx_mul(grad, mask). */                                                                    \
    int fx_dropout_##S(fx_ctx* ctx, const T* x, T* mask, T* y, int64_t n, double p, uint64_t seed);                    \
    /* Bias gradient out[c] = sum over (o, i) of g[o, c, i]: reduce_gradient_for_broadcasting,                         \
       src/ops/basic.rs:10-53 (three axis sums for a conv bias) in one pass; fixed summation order per shape. */       \
    int fx_bias_grad_##S(fx_ctx* ctx, const T* g, T* out, int64_t outer, int64_t C, int64_t inner);                    \
    /* ReLU::gradient (ops/unary.rs:358-375, mask taken from the activation's output y: y > 0 exactly when its input   \
       was) followed by that bias gradient, in one pass: gm = g * (y > 0) is written for the weight / data gradients   \
       and dbias[c] = sum of gm over (o, i).  gm has the bits of fx_relu_bwd(g, y); dbias is summed in a fixed order   \
       of its own (equal to fx_bias_grad(gm) up to rounding). */                                                       \
    int fx_relu_bwd_bias_grad_##S(fx_ctx* ctx, const T* g, const T* y, T* gm, T* dbias, int64_t outer, int64_t C,      \
                                  int64_t inner);                                                                      \
    /* CCELoss with mean reduction, src/nn/losses/classification.rs:191-257: probs[B,C] = softmax(logits) (kept for    \
       the backward), loss[1] = mean_b( -sum_c targets*log(clamp(probs, 1e-8, 1-1e-8)) ).  bwd: d logits from the      \
       upstream gradient of the loss (1 element on the device) through Mean, Neg, Sum, Mul, Log, Clamp and the         \
       softmax Jacobian (src/ops/batched.rs:106-131). */                                                               \
    int fx_softmax_ce_fwd_##S(fx_ctx* ctx, const T* logits, const T* targets, T* probs, T* loss, int64_t B, int64_t C); \
    int fx_softmax_ce_bwd_##S(fx_ctx* ctx, const T* probs, const T* targets, const T* grad_loss, T* dlogits, int64_t B, \
                              int64_t C);                                                                              \
    /* The forward pass plus d logits for an upstream gradient of exactly 1 -- what backward() seeds a scalar loss     \
       with (src/graph/mod.rs:700-733) -- in the same launch(es): probs and loss have the bits of fx_softmax_ce_fwd,   \
       dlogits those of fx_softmax_ce_bwd on a device 1.  For a training step whose loss is the root of the tape. */   \
    int fx_softmax_ce_fwd_unit_grad_##S(fx_ctx* ctx, const T* logits, const T* targets, T* probs, T* loss, T* dlogits, \
                                        int64_t B, int64_t C);                                                         \
    /* Adam::step for one parameter, in place on p, m, v (src/nn/optim/adam.rs:288-358, no amsgrad):                   \
       m = m*b1 + g*(1-b1); v = v*b2 + (g*g)*(1-b2); p = p - ((m/bc1)/(sqrt(v/bc2)+eps))*lr [- p*(wd*lr)], with        \
       bc1 = 1-max(b1^t,1e-8), bc2 = 1-max(b2^t,1e-8) computed by the caller (adam.rs:110-126).  Same operations in    \
       the same order as the composed kernels: bit-identical results. */                                               \
    int fx_adam_step_##S(fx_ctx* ctx, T* p, const T* g, T* m, T* v, int64_t n, T lr, T beta1, T beta2, T eps,          \
                         T weight_decay, T bc1, T bc2);                                                                \
    /* The same step with AMSGrad (adam.rs:203-221, 326-338): vmax = max(vmax, v) elementwise (a >= b ? a : b,         \
       cpu.rs:717-739) after v is updated, and vmax takes v's place in the denominator; in place on vmax too. */        \
    int fx_adam_amsgrad_step_##S(fx_ctx* ctx, T* p, const T* g, T* m, T* v, T* vmax, int64_t n, T lr, T beta1, T beta2, \
                                 T eps, T weight_decay, T bc1, T bc2);                                                 \
    /* SGD::step without momentum or weight decay, src/nn/optim/sgd.rs:210-245: p = p - g*lr, in place. */             \
    int fx_sgd_step_##S(fx_ctx* ctx, T* p, const T* g, int64_t n, T lr);                                               \
    /* SGD::step in full (sgd.rs:128-245): e = g + p*weight_decay when weight_decay != 0 (L2, apply_weight_decay);     \
       momentum != 0: buf = buf*momentum + e (update_momentum_buffer; a new buffer starts at zero) and the update is   \
       buf, or buf*momentum + e with nesterov; p = p - update*lr.  buf must be NULL exactly when momentum == 0.        \
       Composed order, bit-identical to the op-by-op path. */                                                          \
    int fx_sgd_momentum_step_##S(fx_ctx* ctx, T* p, const T* g, T* buf, int64_t n, T lr, T momentum, T weight_decay,   \
                                 int nesterov);                                                                        \
    /* The same updates for `count` parameters in one launch (the optimizers' loop over a parameter group,             \
       adam.rs:288-358 / sgd.rs:210-245): p, g, m, v, vmax, buf, n are HOST arrays of `count` device pointers /        \
       element counts; element arithmetic and results are those of the one-tensor calls. */                            \
    int fx_adam_step_multi_##S(fx_ctx* ctx, int count, T* const* p, const T* const* g, T* const* m, T* const* v,       \
                               const int64_t* n, T lr, T beta1, T beta2, T eps, T weight_decay, T bc1, T bc2);         \
    int fx_adam_amsgrad_step_multi_##S(fx_ctx* ctx, int count, T* const* p, const T* const* g, T* const* m,            \
                                       T* const* v, T* const* vmax, const int64_t* n, T lr, T beta1, T beta2, T eps,   \
                                       T weight_decay, T bc1, T bc2);                                                  \
    /* The multi-tensor Adam step for recorded steps (fx_graph_*): the bias corrections, the only scalars of a step    \
       that change from one step to the next, are read from memory the device can address, bc = {bc1, bc2}: device    \
       memory, or page-locked host memory from fx_host_alloc, which the kernel reads in place (the host then rewrites  \
       the two values between launches, once the launch before has finished).  vmax may be NULL (no AMSGrad).  Same    \
       arithmetic and bits as the calls above. */                                                                      \
    int fx_adam_step_multi_bc_##S(fx_ctx* ctx, int count, T* const* p, const T* const* g, T* const* m, T* const* v,    \
                                  T* const* vmax, const int64_t* n, T lr, T beta1, T beta2, T eps, T weight_decay,     \
                                  const T* bc);                                                                        \
    int fx_sgd_step_multi_##S(fx_ctx* ctx, int count, T* const* p, const T* const* g, const int64_t* n, T lr);         \
    int fx_sgd_momentum_step_multi_##S(fx_ctx* ctx, int count, T* const* p, const T* const* g, T* const* buf,          \
                                       const int64_t* n, T lr, T momentum, T weight_decay, int nesterov);

FX_DECLARE_KERNELS(float, f32)
FX_DECLARE_KERNELS(double, f64)

/* ---- recorded steps (HIP graphs) -------------------------------------------------------------------------------
 * No counterpart in the reference, which launches every kernel of a training step from the host
 * (examples/common/training.rs:105-160; about 230 launches in the CNN configuration, 3.4 us each, more than the kernels
 * themselves take).  Between fx_graph_begin and fx_graph_end the context's stream RECORDS the calls made on this
 * context instead of running them; fx_graph_launch then replays the recording as one submission, with the pointer and
 * scalar arguments of the recording.  Rules for the recorded region:
 *   - run the same calls once eagerly first: the pool then serves every request from its buckets, the library's
 *     scratch region has its final size and the convolution tile shapes are timed (none of this can happen while
 *     recording: fx_alloc may still fall through to hipMalloc, but a call that waits for the stream -- fx_sync,
 *     fx_h2d, fx_d2h, fx_timer_stop, fx_pool_cleanup, the tile timing -- makes fx_graph_end fail);
 *   - blocks released with fx_free while recording stay out of the pool: they are the graph's temporaries, used at the
 *     same addresses by every launch, and go back to the pool in fx_graph_destroy;
 *   - what a launch reads from outside (the batch) must sit at the recorded addresses: copy new data there;
 *   - scalars that change per step must come from memory: fx_adam_step_multi_bc reads its bias corrections through a
 *     pointer, which may be page-locked host memory (fx_host_alloc) that the host rewrites between launches; an
 *     fx_h2d_async from such memory is recorded as "copy from this host address" and serves larger data the same way.
 * A launch is stream-ordered like any other call; results are bit-identical to the eager calls (same kernels, same
 * arguments). */
/* Which kernel family the last convolution call on this context ran, as a fixed string: "LDS patch (cpk)", "LDS patch, row
 * segments (wgp)", "image layer, row bands (csc)", "stride-2 patch (dg2)", "1x1 as batched slab GEMM (glk)", "implicit GEMM",
 * "implicit GEMM by pixel classes", "explicit GEMM + col2im (CPU-literal mode)", ...  A call that returned an error leaves the
 * previous value.  No counterpart in the reference (KernelManager looks kernels up by name, src/backend/cuda/kernels.rs:223-292):
 * it lets a caller see when a layer shape falls off the specialised kernels onto the implicit GEMM. */
const char* fx_conv2d_last_path(fx_ctx* ctx);
/* 1 when fx_conv2d_wgrad_relu_bias (kind FX_CONV_WGRAD) / fx_conv2d_dgrad_relu (kind FX_CONV_DGRAD) has a fused kernel
 * for this dtype and shape on this context's device (16-byte aligned tensors assumed), else 0. */
int fx_conv2d_bwd_relu_supported(fx_ctx* ctx, int kind, int dtype, int64_t B, int64_t Cin, int64_t H, int64_t W, int64_t Cout,
                                 int64_t kh, int64_t kw, int64_t sh, int64_t sw, int64_t ph, int64_t pw);

typedef struct fx_graph fx_graph;
int fx_graph_begin(fx_ctx* ctx);
int fx_graph_end(fx_ctx* ctx, fx_graph** out);
int fx_graph_launch(fx_ctx* ctx, fx_graph* graph);
/* number of nodes, of kernel nodes, and of pool blocks the graph keeps (any pointer may be NULL) */
int fx_graph_info(fx_graph* graph, int64_t* nodes, int64_t* kernel_nodes, int64_t* held_blocks);
int fx_graph_destroy(fx_ctx* ctx, fx_graph* graph);
/* The library's own scratch region (split-K partials, weight images, reduction partials): its address and size, the
 * number of outgrown regions kept alive for recorded graphs, and the number of live graphs (any pointer may be NULL).
 * A recorded graph holds the scratch address of its recording.  While a graph made by fx_graph_end has not been
 * destroyed, a later eager call that needs a larger region allocates a new one and PARKS the old one (it stays valid
 * for the graph's launches) instead of freeing it; parked regions are freed when the last graph is destroyed or with
 * the context.  Host-only query: it never touches the stream. */
int fx_scratch_info(fx_ctx* ctx, void** current, int64_t* bytes, int64_t* parked_regions, int64_t* live_graphs);
/* Free and total device memory as the driver reports it (hipMemGetInfo); either pointer may be NULL.  No counterpart
 * in the reference: callers use it to check that a call allocated nothing. */
int fx_device_mem_info(fx_ctx* ctx, int64_t* free_bytes, int64_t* total_bytes);
/* Page-locked host memory and an upload from it that does not wait (fx_h2d waits for the copy). */
int fx_host_alloc(fx_ctx* ctx, int64_t bytes, void** out);
int fx_host_free(fx_ctx* ctx, void* ptr);
int fx_h2d_async(fx_ctx* ctx, void* dst, const void* src_pinned, int64_t bytes);

/* ---- an entry point that allocates nothing ---------------------------------------------------------------
 * No counterpart in the reference.  It is for callers that cannot allocate device memory at the time of the call:
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  Same arguments, kernels and
 * results (bit for bit) as fx_reduce_max_f32, but the partial maxima / indices of a reduction whose axis is split
 * across blocks go to a fixed array of FX_NOALLOC_SCRATCH_BYTES inside the library's device image (resolved once per
 * device by fx_init) instead of the context's growing hipMalloc'ed scratch.  A shape whose partials do not fit
 * returns FX_ERR_UNSUPPORTED with the sizes in the message ([8192, 8192] along either axis or as one run needs at
 * most 2.4 MB).  Nothing in the array has to start at zero (every partial is written before it is read), so it
 * is never cleared; all calls on one GPU share it, so calls that overlap on one GPU -- two contexts, or two
 * streams -- race and must be serialised by the caller. */
#define FX_NOALLOC_SCRATCH_BYTES (4 << 20)
int fx_reduce_max_noalloc_f32(fx_ctx* ctx, const float* in, float* out, int64_t* idx_out, int64_t outer, int64_t axis,
                              int64_t inner);

#ifdef __cplusplus
}
#endif
#endif /* FERROX_HIP_H */
