// src/backend/hip/mod.rs -- device context, dtype dispatch and the owning device buffer of the HIP backend.
//
// Replaces src/backend/cuda/{context.rs, ops.rs, kernels.rs, stream_manager.rs} and src/backend/memory/cuda.rs of the
// CUDA backend: the context, the pool and every kernel live behind the C ABI of libferrox_hip.so (`ferrox-hip-sys`).
//   CudaContextManager (cuda/context.rs:30-175)  -> HipContext (fx_init / fx_sync / copies)
//   CudaMemoryPool     (memory/cuda.rs:20-202)   -> fx_alloc / fx_free / fx_pool_* (statistics via `pool_stats`)
//   CudaTensor<T>      (cuda/context.rs:284-763) -> HipTensor<T>: one pool block + shape, returned to the pool on drop
//   DeviceRepr + ValidAsZeroBits (cudarc)        -> HipRepr: picks the _f32 / _f64 entry points
use crate::backend::memory::PoolConfig;
use ferrox_hip_sys as sys;
use ndarray::ArrayD;
use std::os::raw::{c_int, c_void};
use std::sync::{Arc, OnceLock};

/// Element types the library has kernels for.  `unsafe`: the implementor promises that `DTYPE` names its own layout.
pub unsafe trait HipRepr: Copy + Send + Sync + 'static {
    const DTYPE: c_int;
    unsafe fn fx_fill(ctx: *mut sys::fx_ctx, out: *mut Self, v: Self, n: i64) -> c_int;
    unsafe fn fx_fill_normal(ctx: *mut sys::fx_ctx, out: *mut Self, n: i64, seed: u64, mean: Self, std: Self) -> c_int;
    unsafe fn fx_materialize(ctx: *mut sys::fx_ctx, inp: *const Self, out: *mut Self, shape: *const i64, strides: *const i64, ndim: c_int, n: i64) -> c_int;
    unsafe fn fx_binary(ctx: *mut sys::fx_ctx, op: c_int, a: *const Self, b: *const Self, out: *mut Self, n: i64) -> c_int;
    unsafe fn fx_scalar(ctx: *mut sys::fx_ctx, op: c_int, a: *const Self, s: Self, out: *mut Self, n: i64) -> c_int;
    unsafe fn fx_unary(ctx: *mut sys::fx_ctx, op: c_int, a: *const Self, out: *mut Self, n: i64) -> c_int;
    unsafe fn fx_clamp(ctx: *mut sys::fx_ctx, a: *const Self, lo: Self, hi: Self, out: *mut Self, n: i64) -> c_int;
    unsafe fn fx_in_range(ctx: *mut sys::fx_ctx, a: *const Self, lo: Self, hi: Self, out: *mut Self, n: i64) -> c_int;
    unsafe fn fx_softmax_axis(ctx: *mut sys::fx_ctx, inp: *const Self, out: *mut Self, outer: i64, axis: i64, inner: i64) -> c_int;
    unsafe fn fx_reduce_sum(ctx: *mut sys::fx_ctx, inp: *const Self, out: *mut Self, outer: i64, axis: i64, inner: i64) -> c_int;
    unsafe fn fx_reduce_max(ctx: *mut sys::fx_ctx, inp: *const Self, out: *mut Self, idx: *mut i64, outer: i64, axis: i64, inner: i64) -> c_int;
    unsafe fn fx_reduce_min(ctx: *mut sys::fx_ctx, inp: *const Self, out: *mut Self, idx: *mut i64, outer: i64, axis: i64, inner: i64) -> c_int;
    unsafe fn fx_gemm(ctx: *mut sys::fx_ctx, ta: c_int, tb: c_int, m: i64, n: i64, k: i64, a: *const Self, b: *const Self, c: *mut Self) -> c_int;
    unsafe fn fx_conv2d_fwd(ctx: *mut sys::fx_ctx, x: *const Self, w: *const Self, y: *mut Self, d: &[i64; 11]) -> c_int;
    unsafe fn fx_conv2d_dgrad(ctx: *mut sys::fx_ctx, g: *const Self, w: *const Self, dx: *mut Self, d: &[i64; 11], mode: c_int) -> c_int;
    unsafe fn fx_conv2d_wgrad(ctx: *mut sys::fx_ctx, x: *const Self, g: *const Self, dw: *mut Self, d: &[i64; 11], mode: c_int) -> c_int;
    unsafe fn fx_pool2d(ctx: *mut sys::fx_ctx, is_max: bool, inp: *const Self, out: *mut Self, d: &[i64; 10]) -> c_int;
    unsafe fn fx_unpool2d(ctx: *mut sys::fx_ctx, is_max: bool, g: *const Self, x: *const Self, pooled: *const Self, gi: *mut Self, d: &[i64; 10]) -> c_int;
}

macro_rules! impl_hip_repr {
    ($t:ty, $code:expr, $fill:ident, $fill_normal:ident, $materialize:ident, $binary:ident, $scalar:ident, $unary:ident, $clamp:ident,
     $in_range:ident, $softmax:ident, $rsum:ident, $rmax:ident, $rmin:ident, $gemm:ident, $fwd:ident, $dgrad:ident, $wgrad:ident,
     $maxpool:ident, $avgpool:ident, $max_unpool:ident, $avg_unpool:ident) => {
        unsafe impl HipRepr for $t {
            const DTYPE: c_int = $code;
            unsafe fn fx_fill(ctx: *mut sys::fx_ctx, out: *mut Self, v: Self, n: i64) -> c_int { sys::$fill(ctx, out, v, n) }
            unsafe fn fx_fill_normal(ctx: *mut sys::fx_ctx, out: *mut Self, n: i64, seed: u64, mean: Self, std: Self) -> c_int {
                sys::$fill_normal(ctx, out, n, seed, mean, std)
            }
            unsafe fn fx_materialize(ctx: *mut sys::fx_ctx, inp: *const Self, out: *mut Self, shape: *const i64, strides: *const i64, ndim: c_int, n: i64) -> c_int {
                sys::$materialize(ctx, inp, out, shape, strides, ndim, n)
            }
            unsafe fn fx_binary(ctx: *mut sys::fx_ctx, op: c_int, a: *const Self, b: *const Self, out: *mut Self, n: i64) -> c_int { sys::$binary(ctx, op, a, b, out, n) }
            unsafe fn fx_scalar(ctx: *mut sys::fx_ctx, op: c_int, a: *const Self, s: Self, out: *mut Self, n: i64) -> c_int { sys::$scalar(ctx, op, a, s, out, n) }
            unsafe fn fx_unary(ctx: *mut sys::fx_ctx, op: c_int, a: *const Self, out: *mut Self, n: i64) -> c_int { sys::$unary(ctx, op, a, out, n) }
            unsafe fn fx_clamp(ctx: *mut sys::fx_ctx, a: *const Self, lo: Self, hi: Self, out: *mut Self, n: i64) -> c_int { sys::$clamp(ctx, a, lo, hi, out, n) }
            unsafe fn fx_in_range(ctx: *mut sys::fx_ctx, a: *const Self, lo: Self, hi: Self, out: *mut Self, n: i64) -> c_int { sys::$in_range(ctx, a, lo, hi, out, n) }
            unsafe fn fx_softmax_axis(ctx: *mut sys::fx_ctx, inp: *const Self, out: *mut Self, outer: i64, axis: i64, inner: i64) -> c_int {
                sys::$softmax(ctx, inp, out, outer, axis, inner)
            }
            unsafe fn fx_reduce_sum(ctx: *mut sys::fx_ctx, inp: *const Self, out: *mut Self, outer: i64, axis: i64, inner: i64) -> c_int {
                sys::$rsum(ctx, inp, out, outer, axis, inner)
            }
            unsafe fn fx_reduce_max(ctx: *mut sys::fx_ctx, inp: *const Self, out: *mut Self, idx: *mut i64, outer: i64, axis: i64, inner: i64) -> c_int {
                sys::$rmax(ctx, inp, out, idx, outer, axis, inner)
            }
            unsafe fn fx_reduce_min(ctx: *mut sys::fx_ctx, inp: *const Self, out: *mut Self, idx: *mut i64, outer: i64, axis: i64, inner: i64) -> c_int {
                sys::$rmin(ctx, inp, out, idx, outer, axis, inner)
            }
            unsafe fn fx_gemm(ctx: *mut sys::fx_ctx, ta: c_int, tb: c_int, m: i64, n: i64, k: i64, a: *const Self, b: *const Self, c: *mut Self) -> c_int {
                sys::$gemm(ctx, ta, tb, m, n, k, a, b, c)
            }
            unsafe fn fx_conv2d_fwd(ctx: *mut sys::fx_ctx, x: *const Self, w: *const Self, y: *mut Self, d: &[i64; 11]) -> c_int {
                sys::$fwd(ctx, x, w, y, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8], d[9], d[10], std::ptr::null_mut(), 0)
            }
            unsafe fn fx_conv2d_dgrad(ctx: *mut sys::fx_ctx, g: *const Self, w: *const Self, dx: *mut Self, d: &[i64; 11], mode: c_int) -> c_int {
                sys::$dgrad(ctx, g, w, dx, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8], d[9], d[10], mode, std::ptr::null_mut(), 0)
            }
            unsafe fn fx_conv2d_wgrad(ctx: *mut sys::fx_ctx, x: *const Self, g: *const Self, dw: *mut Self, d: &[i64; 11], mode: c_int) -> c_int {
                sys::$wgrad(ctx, x, g, dw, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8], d[9], d[10], mode, std::ptr::null_mut(), 0)
            }
            unsafe fn fx_pool2d(ctx: *mut sys::fx_ctx, is_max: bool, inp: *const Self, out: *mut Self, d: &[i64; 10]) -> c_int {
                if is_max { sys::$maxpool(ctx, inp, out, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8], d[9]) }
                else { sys::$avgpool(ctx, inp, out, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8], d[9]) }
            }
            unsafe fn fx_unpool2d(ctx: *mut sys::fx_ctx, is_max: bool, g: *const Self, x: *const Self, pooled: *const Self, gi: *mut Self, d: &[i64; 10]) -> c_int {
                if is_max { sys::$max_unpool(ctx, g, x, pooled, gi, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8], d[9]) }
                else { sys::$avg_unpool(ctx, g, gi, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8], d[9]) }
            }
        }
    };
}
impl_hip_repr!(f32, sys::FX_F32, fx_fill_f32, fx_fill_normal_f32, fx_materialize_f32, fx_binary_f32, fx_scalar_f32, fx_unary_f32, fx_clamp_f32,
               fx_in_range_f32, fx_softmax_axis_f32, fx_reduce_sum_f32, fx_reduce_max_f32, fx_reduce_min_f32, fx_gemm_f32, fx_conv2d_fwd_f32,
               fx_conv2d_dgrad_f32, fx_conv2d_wgrad_f32, fx_maxpool2d_f32, fx_avgpool2d_f32, fx_max_unpool2d_f32, fx_avg_unpool2d_f32);
impl_hip_repr!(f64, sys::FX_F64, fx_fill_f64, fx_fill_normal_f64, fx_materialize_f64, fx_binary_f64, fx_scalar_f64, fx_unary_f64, fx_clamp_f64,
               fx_in_range_f64, fx_softmax_axis_f64, fx_reduce_sum_f64, fx_reduce_max_f64, fx_reduce_min_f64, fx_gemm_f64, fx_conv2d_fwd_f64,
               fx_conv2d_dgrad_f64, fx_conv2d_wgrad_f64, fx_maxpool2d_f64, fx_avgpool2d_f64, fx_max_unpool2d_f64, fx_avg_unpool2d_f64);

/// One device, one compute stream, one pool per dtype; shared by the f32 and f64 `BackendManager`s.
pub struct HipContext {
    raw: *mut sys::fx_ctx,
    /// 0 = mathematical conv gradients (what the reference's CUDA kernels compute);
    /// 1 = the CPU backend's literal arithmetic (flat re-read of grad_output, batch-major col2im)
    pub conv_grad_mode: c_int,
}
// The library serialises allocator calls and launches per context and makes the device current on every call.
unsafe impl Send for HipContext {}
unsafe impl Sync for HipContext {}

static HIP_CONTEXT: OnceLock<Option<HipContext>> = OnceLock::new();

/// PoolConfig (memory/mod.rs:15-82) -> fx_pool_config with the reference's allocation policy.  `to_be_evicted()` and
/// `eviction_threshold()` are the two `pub(crate)` getters rust/PATCHES.md adds to BucketConfig (the fields are private).
pub fn pool_config_to_ffi(cfg: &PoolConfig) -> sys::fx_pool_config {
    let empty = sys::fx_bucket_config { min_elems: 0, max_elems: 0, max_blocks: 0, to_evict: 0, eviction_threshold_ms: -1 };
    let mut out = sys::fx_pool_config { n_buckets: 0, literal_ids: 0, best_fit: 0, reserved: 0, buckets: [empty; sys::FX_MAX_BUCKETS] };
    for (i, b) in cfg.bucket_configs.iter().take(sys::FX_MAX_BUCKETS).enumerate() {
        out.buckets[i] = sys::fx_bucket_config {
            min_elems: b.min_size as i64,
            max_elems: if b.max_size == usize::MAX { i64::MAX } else { b.max_size as i64 },
            max_blocks: b.max_allocations as i64,
            to_evict: b.to_be_evicted() as i64,
            eviction_threshold_ms: b.eviction_threshold().map(|ms| ms as i64).unwrap_or(-1),
        };
        out.n_buckets = (i + 1) as i32;
    }
    out
}

impl HipContext {
    /// CudaContextManager::from_device_id (cuda/context.rs:35-59).  `pool = None` takes the library's default pool
    /// (best fit, block counts sized for 288 GB of HBM).
    pub fn init(device: usize, pool: Option<&PoolConfig>) -> Result<HipContext, String> {
        let mut raw: *mut sys::fx_ctx = std::ptr::null_mut();
        let ffi_cfg = pool.map(pool_config_to_ffi);
        let cfg_ptr = ffi_cfg.as_ref().map(|c| c as *const sys::fx_pool_config).unwrap_or(std::ptr::null());
        sys::check(unsafe { sys::fx_init(device as c_int, cfg_ptr, &mut raw) })?;
        Ok(HipContext { raw, conv_grad_mode: 0 })
    }
    pub fn raw(&self) -> *mut sys::fx_ctx { self.raw }
    pub fn synchronize(&self) -> Result<(), String> { sys::check(unsafe { sys::fx_sync(self.raw) }) }
    pub fn name(&self) -> String {
        let mut buf = [0 as std::os::raw::c_char; 256];
        if unsafe { sys::fx_device_name(self.raw, buf.as_mut_ptr(), buf.len() as i64) } != sys::FX_OK {
            return "unknown".to_string();
        }
        unsafe { std::ffi::CStr::from_ptr(buf.as_ptr()) }.to_string_lossy().into_owned()
    }
    /// PoolStats (memory/mod.rs:195-202) of one dtype's pool.
    pub fn pool_stats<T: HipRepr>(&self) -> Result<sys::fx_pool_stats, String> {
        let mut st: sys::fx_pool_stats = unsafe { std::mem::zeroed() };
        sys::check(unsafe { sys::fx_pool_stats_get(self.raw, T::DTYPE, &mut st) })?;
        Ok(st)
    }
    pub fn pool_cleanup<T: HipRepr>(&self) -> Result<(), String> { sys::check(unsafe { sys::fx_pool_cleanup(self.raw, T::DTYPE) }) }
    pub fn pool_reset<T: HipRepr>(&self) -> Result<(), String> { sys::check(unsafe { sys::fx_pool_reset(self.raw, T::DTYPE) }) }
}

impl Drop for HipContext {
    fn drop(&mut self) {
        unsafe { sys::fx_destroy(self.raw) };
    }
}

/// Process-wide context, created on first use on device 0 (BackendManager::init calls `init_hip_context` first when a
/// pool configuration was given).  `None` when no gfx950 device is present.
pub fn init_hip_context(device: usize, pool: Option<&PoolConfig>) -> bool {
    HIP_CONTEXT.get_or_init(|| HipContext::init(device, pool).ok()).is_some()
}
pub fn hip_context() -> Result<&'static HipContext, String> {
    HIP_CONTEXT
        .get_or_init(|| HipContext::init(0, None).ok())
        .as_ref()
        .ok_or_else(|| "CUDA backend not available".to_string()) // wording of with_cuda_context, manager.rs:405-416
}
/// with_cuda_context / with_cuda_ops of manager.rs:405-431
pub fn with_hip<R>(f: impl FnOnce(&HipContext) -> Result<R, String>) -> Result<R, String> {
    f(hip_context()?)
}

/// One block of the pool.  It goes back to the pool when its last owner lets go (CudaTensor::drop, cuda/context.rs:726-742).
#[derive(Debug)]
struct HipBlock<T: HipRepr> {
    ptr: *mut T,
    granted: i64,
    id: u64,
}
unsafe impl<T: HipRepr> Send for HipBlock<T> {}
unsafe impl<T: HipRepr> Sync for HipBlock<T> {}

impl<T: HipRepr> Drop for HipBlock<T> {
    /// A failure is ignored, as in the reference.
    fn drop(&mut self) {
        if let Ok(ctx) = hip_context() {
            unsafe { sys::fx_free(ctx.raw(), T::DTYPE, self.block.ptr as *mut c_void, self.id) };
        }
    }
}

/// A counted reference to a pool block plus a shape: the device half of a tensor.  Always contiguous (views are materialised
/// eagerly, like CUDAStorage does, storage/cuda.rs:795-911).  No method of the storage trait writes a block after the call that
/// produced it has returned (every op returns new storage; the `&mut self` view methods, storage/mod.rs:246-269, materialise into a
/// new block), so `share()` -- a second owner of the same block -- cannot be told from the device copy of `try_clone()`.
#[derive(Debug)]
pub struct HipTensor<T: HipRepr> {
    block: Arc<HipBlock<T>>,
    shape: Vec<usize>,
}

impl<T: HipRepr> HipTensor<T> {
    /// CudaOps::get_tensor (cuda/ops.rs:121-133): the block comes from the pool and is NOT cleared.
    pub fn alloc(shape: &[usize]) -> Result<Self, String> {
        let n: usize = shape.iter().product();
        let ctx = hip_context()?;
        let (mut p, mut granted, mut id) = (std::ptr::null_mut::<c_void>(), 0i64, 0u64);
        sys::check(unsafe { sys::fx_alloc(ctx.raw(), T::DTYPE, n as i64, &mut p, &mut granted, &mut id) })?;
        Ok(HipTensor { block: Arc::new(HipBlock { ptr: p as *mut T, granted, id }), shape: shape.to_vec() })
    }
    pub fn full(shape: &[usize], value: T) -> Result<Self, String> {
        let t = Self::alloc(shape)?;
        sys::check(unsafe { T::fx_fill(hip_context()?.raw(), t.block.ptr, value, t.size() as i64) })?;
        Ok(t)
    }
    /// host_to_device, cuda/context.rs:81-97
    pub fn from_slice(data: &[T], shape: &[usize]) -> Result<Self, String> {
        let t = Self::alloc(shape)?;
        if data.len() != t.size() {
            return Err(format!("Data length {} doesn't match shape {:?}", data.len(), shape));
        }
        let bytes = (data.len() * std::mem::size_of::<T>()) as i64;
        sys::check(unsafe { sys::fx_h2d(hip_context()?.raw(), t.block.ptr as *mut c_void, data.as_ptr() as *const c_void, bytes) })?;
        Ok(t)
    }
    /// CudaTensor::from_cpu_array, cuda/context.rs:330-351
    pub fn from_cpu_array(array: &ArrayD<T>) -> Result<Self, String> {
        let owned;
        let data: &[T] = match array.as_slice() {
            Some(s) => s,
            None => {
                owned = array.iter().copied().collect::<Vec<T>>();
                &owned
            }
        };
        Self::from_slice(data, array.shape())
    }
    /// CudaTensor::to_vec, cuda/context.rs:410-426 (an oversized pooled block is truncated to the tensor's size)
    pub fn to_vec(&self) -> Result<Vec<T>, String> {
        let n = self.size();
        let mut v = Vec::<T>::with_capacity(n);
        let bytes = (n * std::mem::size_of::<T>()) as i64;
        sys::check(unsafe { sys::fx_d2h(hip_context()?.raw(), v.as_mut_ptr() as *mut c_void, self.block.ptr as *const c_void, bytes) })?;
        unsafe { v.set_len(n) };
        Ok(v)
    }
    /// CudaTensor::clone, cuda/context.rs:744-763: a device-to-device copy into a new pool block.
    pub fn try_clone(&self) -> Result<Self, String> {
        let t = Self::alloc(&self.shape)?;
        let bytes = (self.size() * std::mem::size_of::<T>()) as i64;
        sys::check(unsafe { sys::fx_d2d(hip_context()?.raw(), t.block.ptr as *mut c_void, self.block.ptr as *const c_void, bytes) })?;
        Ok(t)
    }
    /// A second owner of the same block (what `clone_storage` hands out: 61 device copies per CNN training step become
    /// reference-count bumps).  Callers that do write blocks in place (fused optimizer steps, a recorded step's batch) must use
    /// `try_clone()` for anything that has to keep its old value.
    pub fn share(&self) -> Self {
        HipTensor { block: Arc::clone(&self.block), shape: self.shape.clone() }
    }
    pub fn shape(&self) -> &[usize] { &self.shape }
    pub fn size(&self) -> usize { self.shape.iter().product() }
    pub fn ndim(&self) -> usize { self.shape.len() }
    pub fn ptr(&self) -> *const T { self.block.ptr }
    pub fn ptr_mut(&self) -> *mut T { self.block.ptr }
    pub fn granted_elems(&self) -> i64 { self.block.granted }
    /// Metadata-only reshape (the storage is contiguous).
    pub fn set_shape(&mut self, shape: Vec<usize>) { self.shape = shape; }
}

impl<T: HipRepr> Clone for HipTensor<T> {
    fn clone(&self) -> Self { self.try_clone().expect("device-to-device copy failed") }
}

