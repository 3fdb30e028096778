// src/backend/storage/hip.rs -- `HipStorage<T>`: the MI355X implementation of `trait StorageBackend<T>`
// (src/backend/storage/mod.rs:24-422).  It takes the place of `CUDAStorage<T>` (src/backend/storage/cuda.rs:28-1381):
// same method set, same ownership (every compute method returns new owned storage, view methods work in place and
// materialise eagerly), the reference's error strings; every kernel is one call into libferrox_hip.so.
use super::StorageBackend;
use crate::backend::hip::{hip_context, HipRepr, HipTensor};
use crate::backend::{FerroxCudaF, FerroxCudaN, FerroxF, FerroxN};
use ferrox_hip_sys as sys;
use ndarray::ArrayD;
use std::os::raw::c_int;

#[derive(Debug, Clone)]
pub struct HipStorage<T: FerroxCudaN + HipRepr> {
    pub hip_data: HipTensor<T>,
}

type Boxed<T> = Result<Box<dyn StorageBackend<T>>, String>;

impl<T: FerroxCudaN + HipRepr> HipStorage<T> {
    pub fn new(hip_data: HipTensor<T>) -> Self {
        Self { hip_data }
    }
    fn boxed(t: HipTensor<T>) -> Boxed<T> {
        Ok(Box::new(HipStorage::new(t)))
    }
    fn raw() -> Result<*mut sys::fx_ctx, String> {
        Ok(hip_context()?.raw())
    }
    fn n(&self) -> i64 {
        self.hip_data.size() as i64
    }
    /// The operand as GPU storage, or the reference's error for a mixed-device call.
    fn gpu<'a>(other: &'a dyn StorageBackend<T>, mixed_msg: &str) -> Result<&'a HipStorage<T>, String> {
        if !other.is_gpu() {
            return Err(mixed_msg.to_string());
        }
        other.as_any().downcast_ref::<HipStorage<T>>().ok_or_else(|| "Failed to cast to GPU storage".to_string())
    }
    /// add / sub / mul / div / min / max accept a CPU operand and upload it first (storage/cuda.rs:93-115); comparisons,
    /// powf, matmul and the convolutions refuse a mixed-device call.
    fn binary(&self, op: c_int, other: &dyn StorageBackend<T>, what: &str, upload_cpu: bool) -> Boxed<T> {
        let uploaded;
        let rhs: &HipTensor<T> = if other.is_gpu() {
            let o = other.as_any().downcast_ref::<HipStorage<T>>().ok_or("Failed to cast to GPU storage")?;
            if self.shape() != o.shape() {
                return Err(format!("Shape mismatch for GPU {}: {:?} vs {:?}", what, self.shape(), o.shape()));
            }
            &o.hip_data
        } else if upload_cpu {
            let data = other.cpu_data()?;
            if self.shape() != data.shape() {
                return Err(format!("Shape mismatch for mixed {}: {:?} vs {:?}", what, self.shape(), data.shape()));
            }
            uploaded = HipTensor::from_cpu_array(data)?;
            &uploaded
        } else {
            return Err(format!("GPU-CPU mixed operations not supported for {}", what));
        };
        let out = HipTensor::<T>::alloc(self.shape())?;
        sys::check(unsafe { T::fx_binary(Self::raw()?, op, self.hip_data.ptr(), rhs.ptr(), out.ptr_mut(), self.n()) })?;
        Self::boxed(out)
    }
    fn scalar(&self, op: c_int, s: T) -> Boxed<T> {
        let out = HipTensor::<T>::alloc(self.shape())?;
        sys::check(unsafe { T::fx_scalar(Self::raw()?, op, self.hip_data.ptr(), s, out.ptr_mut(), self.n()) })?;
        Self::boxed(out)
    }
    fn unary(&self, op: c_int) -> Boxed<T> {
        let out = HipTensor::<T>::alloc(self.shape())?;
        sys::check(unsafe { T::fx_unary(Self::raw()?, op, self.hip_data.ptr(), out.ptr_mut(), self.n()) })?;
        Self::boxed(out)
    }
    /// [outer, axis, inner] view of a contiguous shape around `axis`.
    fn oai(shape: &[usize], axis: usize) -> (i64, i64, i64) {
        let outer: usize = shape[..axis].iter().product();
        let inner: usize = shape[axis + 1..].iter().product();
        (outer as i64, shape[axis] as i64, inner as i64)
    }
    /// kind 0 sum, 2 max, 3 min.  One kernel per axis, axes in descending order with a temporary between steps
    /// (CudaOps::reduce_axes, cuda/ops.rs:2171-2284; the CPU backend reduces in the same order, cpu.rs:85-95).
    fn reduce(&self, kind: u8, axes: Option<&[usize]>, keep_dims: bool) -> Result<HipTensor<T>, String> {
        let ctx = Self::raw()?;
        let launch = |inp: *const T, out: *mut T, (outer, ax, inner): (i64, i64, i64)| -> Result<(), String> {
            sys::check(unsafe {
                match kind {
                    0 => T::fx_reduce_sum(ctx, inp, out, outer, ax, inner),
                    2 => T::fx_reduce_max(ctx, inp, out, std::ptr::null_mut(), outer, ax, inner),
                    _ => T::fx_reduce_min(ctx, inp, out, std::ptr::null_mut(), outer, ax, inner),
                }
            })
        };
        let shape = self.shape().to_vec();
        let axes = match axes {
            None => {
                let final_shape: Vec<usize> = if keep_dims { vec![1; shape.len()] } else { vec![] };
                let out = HipTensor::<T>::alloc(&final_shape)?;
                launch(self.hip_data.ptr(), out.ptr_mut(), (1, self.n(), 1))?;
                return Ok(out);
            }
            Some(a) => a,
        };
        if axes.is_empty() {
            return Err("Empty axes list provided".to_string());
        }
        for &a in axes {
            if a >= shape.len() {
                return Err(format!("Axis {} is out of bounds for tensor with {} dimensions", a, shape.len()));
            }
        }
        let mut sorted = axes.to_vec();
        sorted.sort_unstable_by(|a, b| b.cmp(a));
        sorted.dedup();
        let mut final_shape = shape.clone();
        for &a in &sorted {
            if keep_dims { final_shape[a] = 1 } else { final_shape.remove(a); }
        }
        let mut cur = shape;
        let mut held: Option<HipTensor<T>> = None;
        for (i, &a) in sorted.iter().enumerate() {
            let view = Self::oai(&cur, a);
            cur.remove(a);
            let out = HipTensor::<T>::alloc(if i + 1 == sorted.len() { &final_shape } else { &cur })?;
            let src = held.as_ref().map(|t| t.ptr()).unwrap_or(self.hip_data.ptr());
            launch(src, out.ptr_mut(), view)?;
            held = Some(out);
        }
        Ok(held.expect("at least one axis"))
    }
    /// Gather-copy of a strided view of self into a new contiguous block that then replaces self's
    /// (CudaOps::materialize, cuda/ops.rs:175-214; shape and strides travel as host arguments).
    fn materialize_into(&mut self, new_shape: Vec<usize>, strides: Vec<i64>) -> Result<(), String> {
        let out = HipTensor::<T>::alloc(&new_shape)?;
        let sh: Vec<i64> = new_shape.iter().map(|&d| d as i64).collect();
        let n: usize = new_shape.iter().product();
        sys::check(unsafe {
            T::fx_materialize(Self::raw()?, self.hip_data.ptr(), out.ptr_mut(), sh.as_ptr(), strides.as_ptr(), sh.len() as c_int, n as i64)
        })?;
        self.hip_data = out; // the old block returns to the pool
        Ok(())
    }
    fn conv_dims(x: &[usize], w: &[usize], stride: (usize, usize), padding: (usize, usize)) -> [i64; 11] {
        [x[0] as i64, x[1] as i64, x[2] as i64, x[3] as i64, w[0] as i64, w[2] as i64, w[3] as i64,
         stride.0 as i64, stride.1 as i64, padding.0 as i64, padding.1 as i64]
    }
    fn pool(&self, is_max: bool, d: [i64; 10], out_shape: &[usize]) -> Boxed<T> {
        let out = HipTensor::<T>::alloc(out_shape)?;
        sys::check(unsafe { T::fx_pool2d(Self::raw()?, is_max, self.hip_data.ptr(), out.ptr_mut(), &d) })?;
        Self::boxed(out)
    }
    #[allow(clippy::too_many_arguments)]
    fn unpool(is_max: bool, what: &str, grad_output: &dyn StorageBackend<T>, original_input: &dyn StorageBackend<T>,
              pooled_output: &dyn StorageBackend<T>, k: (usize, usize), s: (usize, usize), p: (usize, usize)) -> Boxed<T> {
        if !(grad_output.is_gpu() && original_input.is_gpu() && pooled_output.is_gpu()) {
            return Err(format!("Mixed GPU/CPU {} not supported - move all tensors to same device", what));
        }
        let g = grad_output.as_any().downcast_ref::<HipStorage<T>>().ok_or("Failed to cast grad_output to GPU storage")?;
        let x = original_input.as_any().downcast_ref::<HipStorage<T>>().ok_or("Failed to cast original_input to GPU storage")?;
        let y = pooled_output.as_any().downcast_ref::<HipStorage<T>>().ok_or("Failed to cast pooled_output to GPU storage")?;
        let xs = x.shape();
        let one_d = xs.len() == 3;
        if !one_d && (xs.len() != 4 || g.ndim() != 4) {
            return Err("Unpool2D requires 4D tensors [N, C, H, W]".to_string());
        }
        if one_d && g.ndim() != 3 {
            return Err("Unpool1D requires 3D tensors [N, C, L]".to_string());
        }
        let d = [xs[0] as i64, xs[1] as i64, if one_d { 1 } else { xs[2] as i64 }, xs[if one_d { 2 } else { 3 }] as i64,
                 k.0 as i64, k.1 as i64, s.0 as i64, s.1 as i64, p.0 as i64, p.1 as i64];
        let out = HipTensor::<T>::alloc(xs)?;
        sys::check(unsafe { T::fx_unpool2d(Self::raw()?, is_max, g.hip_data.ptr(), x.hip_data.ptr(), y.hip_data.ptr(), out.ptr_mut(), &d) })?;
        Self::boxed(out)
    }

    // ---- factories used by BackendManager (CUDAStorage::{zeros, ones, full, randn}, storage/cuda.rs:1383-1421) ----
    pub fn zeros(shape: &[usize]) -> Boxed<T> {
        Self::boxed(HipTensor::full(shape, <T as FerroxN>::zero())?)
    }
    pub fn ones(shape: &[usize]) -> Boxed<T> {
        Self::boxed(HipTensor::full(shape, <T as FerroxN>::one())?)
    }
    pub fn full(shape: &[usize], value: T) -> Boxed<T> {
        Self::boxed(HipTensor::full(shape, value)?)
    }
    /// Standard normal values from the library's counter-based generator (seed 1000 like CudaOps::randn's call).
    pub fn randn(shape: &[usize]) -> Boxed<T> {
        let t = HipTensor::<T>::alloc(shape)?;
        sys::check(unsafe { T::fx_fill_normal(Self::raw()?, t.ptr_mut(), t.size() as i64, 1000, <T as FerroxN>::zero(), <T as FerroxN>::one()) })?;
        Self::boxed(t)
    }
    pub fn from_cpu_array(data: &ArrayD<T>) -> Boxed<T> {
        Self::boxed(HipTensor::from_cpu_array(data)?)
    }
    /// GPU -> CPU (BackendManager::move_storage, manager.rs:281-320)
    pub fn to_cpu_array(&self) -> Result<ArrayD<T>, String> {
        let host = self.hip_data.to_vec()?;
        ArrayD::from_shape_vec(ndarray::IxDyn(self.shape()), host).map_err(|e| format!("Failed to create CPU array: {}", e))
    }
}

impl<T> StorageBackend<T> for HipStorage<T>
where
    T: FerroxCudaN + HipRepr + Clone,
{
    fn shape(&self) -> &[usize] {
        self.hip_data.shape()
    }
    fn as_any(&self) -> &dyn std::any::Any {
        self
    }
    fn into_any(self: Box<Self>) -> Box<dyn std::any::Any + 'static> {
        self as Box<dyn std::any::Any + 'static>
    }
    fn ndim(&self) -> usize {
        self.hip_data.shape().len()
    }
    fn size(&self) -> usize {
        self.hip_data.shape().iter().product()
    }
    fn is_gpu(&self) -> bool {
        true
    }
    fn cpu_data(&self) -> Result<&ArrayD<T>, String> {
        Err("Data is on GPU. Use .to_cpu() to move it first".to_string())
    }
    fn cpu_data_mut(&mut self) -> Result<&mut ArrayD<T>, String> {
        Err("Data is on GPU. Use .to_cpu() to move it first".to_string())
    }
    fn owns_data(&self) -> bool {
        true
    }
    /// CudaTensor::clone (cuda/context.rs:744-763) is a device-to-device copy; here the clone is a second owner of the same
    /// block, which the trait cannot tell apart (see HipTensor::share) and which takes the reference's per-node deep clones
    /// (graph/mod.rs:735-751) and `Tensor::clone` (tensor.rs:34-48) out of the training step's device time.
    fn clone_storage(&self) -> Boxed<T> {
        Self::boxed(self.hip_data.share())
    }

    // ---- elementwise (storage/cuda.rs:74-319): a CPU operand is uploaded first ----
    fn add(&self, other: &dyn StorageBackend<T>) -> Boxed<T> {
        self.binary(sys::FX_ADD, other, "addition", true)
    }
    fn sub(&self, other: &dyn StorageBackend<T>) -> Boxed<T> {
        self.binary(sys::FX_SUB, other, "subtraction", true)
    }
    fn mul(&self, other: &dyn StorageBackend<T>) -> Boxed<T> {
        self.binary(sys::FX_MUL, other, "multiplication", true)
    }
    fn div(&self, other: &dyn StorageBackend<T>) -> Boxed<T> {
        self.binary(sys::FX_DIV, other, "division", true)
    }
    fn min(&self, other: &dyn StorageBackend<T>) -> Boxed<T> {
        self.binary(sys::FX_MIN, other, "min operation", true)
    }
    fn max(&self, other: &dyn StorageBackend<T>) -> Boxed<T> {
        self.binary(sys::FX_MAX, other, "max operation", true)
    }
    // scalar ops: the scalar is a kernel argument (the reference fills a full-size temporary first, cuda/ops.rs:435-464)
    fn add_scalar(&self, scalar: T) -> Boxed<T> {
        self.scalar(sys::FX_ADD_SCALAR, scalar)
    }
    fn sub_scalar(&self, scalar: T) -> Boxed<T> {
        self.scalar(sys::FX_SUB_SCALAR, scalar)
    }
    fn mul_scalar(&self, scalar: T) -> Boxed<T> {
        self.scalar(sys::FX_MUL_SCALAR, scalar)
    }
    fn div_scalar(&self, scalar: T) -> Boxed<T> {
        self.scalar(sys::FX_DIV_SCALAR, scalar)
    }
    fn neg(&self) -> Boxed<T> {
        self.unary(sys::FX_NEG)
    }
    fn abs(&self) -> Boxed<T> {
        self.unary(sys::FX_ABS)
    }
    fn sqrt(&self) -> Boxed<T>
    where
        T: FerroxCudaF,
    {
        self.unary(sys::FX_SQRT)
    }
    fn clamp(&self, min_val: T, max_val: T) -> Boxed<T> {
        let out = HipTensor::<T>::alloc(self.shape())?;
        sys::check(unsafe { T::fx_clamp(Self::raw()?, self.hip_data.ptr(), min_val, max_val, out.ptr_mut(), self.n()) })?;
        Self::boxed(out)
    }
    fn reciprocal(&self) -> Boxed<T> {
        self.unary(sys::FX_RECIPROCAL)
    }

    // ---- comparisons (storage/cuda.rs:373-536): GPU operands only; 1.0 / 0.0 results ----
    fn greater(&self, other: &dyn StorageBackend<T>) -> Boxed<T> {
        self.binary(sys::FX_GREATER, other, "comparison operations", false)
    }
    fn greater_equal(&self, other: &dyn StorageBackend<T>) -> Boxed<T> {
        self.binary(sys::FX_GREATER_EQUAL, other, "comparison operations", false)
    }
    fn less(&self, other: &dyn StorageBackend<T>) -> Boxed<T> {
        self.binary(sys::FX_LESS, other, "comparison operations", false)
    }
    fn less_equal(&self, other: &dyn StorageBackend<T>) -> Boxed<T> {
        self.binary(sys::FX_LESS_EQUAL, other, "comparison operations", false)
    }
    fn equal(&self, other: &dyn StorageBackend<T>) -> Boxed<T> {
        self.binary(sys::FX_EQUAL, other, "comparison operations", false)
    }
    fn greater_scalar(&self, scalar: T) -> Boxed<T> {
        self.scalar(sys::FX_GREATER_SCALAR, scalar)
    }
    fn greater_equal_scalar(&self, scalar: T) -> Boxed<T> {
        self.scalar(sys::FX_GREATER_EQUAL_SCALAR, scalar)
    }
    fn less_scalar(&self, scalar: T) -> Boxed<T> {
        self.scalar(sys::FX_LESS_SCALAR, scalar)
    }
    fn less_equal_scalar(&self, scalar: T) -> Boxed<T> {
        self.scalar(sys::FX_LESS_EQUAL_SCALAR, scalar)
    }
    fn logical_not(&self) -> Boxed<T> {
        self.unary(sys::FX_LOGICAL_NOT)
    }
    fn in_range(&self, min_val: T, max_val: T) -> Boxed<T> {
        let out = HipTensor::<T>::alloc(self.shape())?;
        sys::check(unsafe { T::fx_in_range(Self::raw()?, self.hip_data.ptr(), min_val, max_val, out.ptr_mut(), self.n()) })?;
        Self::boxed(out)
    }
    fn sign(&self) -> Boxed<T> {
        self.unary(sys::FX_SIGN)
    }

    // ---- matmul (storage/cuda.rs:539-567; checks of cpu.rs:967-1002) ----
    fn matmul(&self, other: &dyn StorageBackend<T>) -> Boxed<T> {
        let o = Self::gpu(other, "GPU-CPU mixed operations not supported for matrix multiplication")?;
        if self.ndim() != 2 || o.ndim() != 2 {
            return Err("Matrix multiplication requires 2D tensors".to_string());
        }
        let (a, b) = (self.shape(), o.shape());
        if a[1] != b[0] {
            return Err(format!("Matrix multiplication shape mismatch: ({}, {}) @ ({}, {})", a[0], a[1], b[0], b[1]));
        }
        let out = HipTensor::<T>::alloc(&[a[0], b[1]])?;
        sys::check(unsafe {
            T::fx_gemm(Self::raw()?, 0, 0, a[0] as i64, b[1] as i64, a[1] as i64, self.hip_data.ptr(), o.hip_data.ptr(), out.ptr_mut())
        })?;
        Self::boxed(out)
    }

    // ---- activations (storage/cuda.rs:569-606) ----
    fn sigmoid(&self) -> Boxed<T>
    where
        T: FerroxF,
    {
        self.unary(sys::FX_SIGMOID)
    }
    fn relu(&self) -> Boxed<T> {
        self.unary(sys::FX_RELU)
    }
    fn exp(&self) -> Boxed<T>
    where
        T: FerroxCudaF,
    {
        self.unary(sys::FX_EXP)
    }
    fn log(&self) -> Boxed<T>
    where
        T: FerroxCudaF,
    {
        self.unary(sys::FX_LOG)
    }
    fn tanh(&self) -> Boxed<T>
    where
        T: FerroxCudaF,
    {
        self.unary(sys::FX_TANH)
    }
    /// Whole tensor as one row (cpu.rs:1018-1036).
    fn softmax(&self) -> Boxed<T>
    where
        T: FerroxF,
    {
        let out = HipTensor::<T>::alloc(self.shape())?;
        sys::check(unsafe { T::fx_softmax_axis(Self::raw()?, self.hip_data.ptr(), out.ptr_mut(), 1, self.n(), 1) })?;
        Self::boxed(out)
    }
    fn softmax_batched(&self, axis: usize) -> Boxed<T>
    where
        T: FerroxCudaF,
    {
        if axis >= self.ndim() {
            return Err(format!("Softmax axis {} out of bounds for tensor with {} dimensions", axis, self.ndim()));
        }
        let (outer, ax, inner) = Self::oai(self.shape(), axis);
        let out = HipTensor::<T>::alloc(self.shape())?;
        sys::check(unsafe { T::fx_softmax_axis(Self::raw()?, self.hip_data.ptr(), out.ptr_mut(), outer, ax, inner) })?;
        Self::boxed(out)
    }
    fn powf(&self, other: &dyn StorageBackend<T>) -> Boxed<T>
    where
        T: FerroxCudaF,
    {
        self.binary(sys::FX_POW, other, "power operations", false)
    }
    fn power_scalar(&self, scalar: T) -> Boxed<T>
    where
        T: FerroxCudaF,
    {
        self.scalar(sys::FX_POW_SCALAR, scalar)
    }

    // ---- reductions (storage/cuda.rs:638-793) ----
    fn sum(&self, axes: Option<&[usize]>, keep_dims: bool) -> Boxed<T> {
        Self::boxed(self.reduce(0, axes, keep_dims)?)
    }
    /// sum, then one multiplication by T(1/n): the CPU backend's rule (cpu.rs:1193-1221).
    fn mean(&self, axes: Option<&[usize]>, keep_dims: bool) -> Boxed<T> {
        let summed = self.reduce(0, axes, keep_dims)?;
        let count: usize = match axes {
            Some(a) => a.iter().map(|&ax| self.shape()[ax]).product(),
            None => self.size(),
        };
        let inv = <T as FerroxN>::from_f64(1.0 / count as f64).ok_or("Failed to convert the element count")?;
        let out = HipTensor::<T>::alloc(summed.shape())?;
        sys::check(unsafe { T::fx_scalar(Self::raw()?, sys::FX_MUL_SCALAR, summed.ptr(), inv, out.ptr_mut(), summed.size() as i64) })?;
        Self::boxed(out)
    }
    fn max_reduce(&self, axes: Option<&[usize]>, keep_dims: bool) -> Boxed<T> {
        Self::boxed(self.reduce(2, axes, keep_dims)?)
    }
    fn min_reduce(&self, axes: Option<&[usize]>, keep_dims: bool) -> Boxed<T> {
        Self::boxed(self.reduce(3, axes, keep_dims)?)
    }

    // ---- view operations, in place, materialised eagerly (storage/cuda.rs:795-911) ----
    fn broadcast_to(&mut self, target_shape: &[usize]) -> Result<(), String> {
        let cur = self.shape().to_vec();
        if target_shape.len() < cur.len() {
            return Err("Cannot broadcast to smaller number of dimensions".to_string());
        }
        let off = target_shape.len() - cur.len();
        let mut strides = vec![0i64; target_shape.len()];
        let mut stride = 1i64;
        for i in (0..cur.len()).rev() {
            let (c, t) = (cur[i], target_shape[off + i]);
            if c != 1 && c != t {
                return Err(format!("Cannot broadcast dimension {} from size {} to size {}", i, c, t));
            }
            strides[off + i] = if c == 1 { 0 } else { stride };
            stride *= c as i64;
        }
        self.materialize_into(target_shape.to_vec(), strides)
    }
    fn reshape(&mut self, new_shape: &[usize]) -> Result<(), String> {
        let total: usize = self.shape().iter().product();
        let new_total: usize = new_shape.iter().product();
        if total != new_total {
            return Err(format!("Cannot reshape tensor with {} elements to shape with {} elements", total, new_total));
        }
        self.hip_data.set_shape(new_shape.to_vec()); // contiguous storage: metadata only
        Ok(())
    }
    fn transpose(&mut self, axes: Option<&[usize]>) -> Result<(), String> {
        let nd = self.ndim();
        let order: Vec<usize> = match axes {
            Some(a) => {
                if a.len() != nd {
                    return Err(format!("Axes length {} doesn't match tensor dimensions {}", a.len(), nd));
                }
                let mut seen = vec![false; nd];
                for &ax in a {
                    if ax >= nd || seen[ax] {
                        return Err("Invalid axes permutation".to_string());
                    }
                    seen[ax] = true;
                }
                a.to_vec()
            }
            None => {
                if nd <= 1 {
                    return Ok(());
                }
                (0..nd).rev().collect()
            }
        };
        let shape = self.shape().to_vec();
        let mut contiguous = vec![1i64; nd];
        for i in (0..nd.saturating_sub(1)).rev() {
            contiguous[i] = contiguous[i + 1] * shape[i + 1] as i64;
        }
        let new_shape: Vec<usize> = order.iter().map(|&o| shape[o]).collect();
        let strides: Vec<i64> = order.iter().map(|&o| contiguous[o]).collect();
        self.materialize_into(new_shape, strides)
    }
    fn unsqueeze(&mut self, axis: usize) -> Result<(), String> {
        if axis > self.ndim() {
            return Err(format!("Axis {} out of bounds for tensor with {} dimensions", axis, self.ndim()));
        }
        let mut shape = self.shape().to_vec();
        shape.insert(axis, 1);
        self.hip_data.set_shape(shape);
        Ok(())
    }
    fn squeeze(&mut self, axis: Option<usize>) -> Result<(), String> {
        let mut shape = self.shape().to_vec();
        match axis {
            Some(ax) => {
                if ax >= shape.len() {
                    return Err(format!("Axis {} out of bounds for tensor with {} dimensions", ax, shape.len()));
                }
                if shape[ax] != 1 {
                    return Err(format!("Cannot squeeze axis {} with size {}", ax, shape[ax]));
                }
                shape.remove(ax);
            }
            None => {
                shape.retain(|&d| d != 1);
                if shape.is_empty() {
                    shape.push(1);
                }
            }
        }
        self.hip_data.set_shape(shape);
        Ok(())
    }

    // ---- convolution (storage/cuda.rs:913-1020) ----
    fn conv2d(&self, filter: &dyn StorageBackend<T>, stride: (usize, usize), padding: (usize, usize)) -> Boxed<T> {
        let f = Self::gpu(filter, "Mixed GPU/CPU convolution not supported - move both tensors to same device")?;
        let (x, w) = (self.shape(), f.shape());
        if x.len() != 4 || w.len() != 4 {
            return Err("Conv2D requires 4D tensors [batch, channels, height, width]".to_string());
        }
        let d = Self::conv_dims(x, w, stride, padding);
        let oh = (x[2] + 2 * padding.0 - w[2]) / stride.0 + 1;
        let ow = (x[3] + 2 * padding.1 - w[3]) / stride.1 + 1;
        let out = HipTensor::<T>::alloc(&[x[0], w[0], oh, ow])?;
        sys::check(unsafe { T::fx_conv2d_fwd(Self::raw()?, self.hip_data.ptr(), f.hip_data.ptr(), out.ptr_mut(), &d) })?;
        Self::boxed(out)
    }
    /// self is the upstream gradient [B, Cout, oh, ow]; the result is the gradient of the convolution's input.
    fn deconv2d(&self, filter: &dyn StorageBackend<T>, output_shape: &[usize], stride: (usize, usize), padding: (usize, usize)) -> Boxed<T> {
        if output_shape.len() != 4 || filter.shape().len() != 4 || self.shape().len() != 4 {
            return Err("Deconv2D requires 4D tensors [batch, channels, height, width]".to_string());
        }
        let f = Self::gpu(filter, "Mixed GPU/CPU deconvolution not supported - move both tensors to same device")?;
        let d = Self::conv_dims(output_shape, f.shape(), stride, padding);
        let out = HipTensor::<T>::alloc(output_shape)?;
        let mode = hip_context()?.conv_grad_mode;
        sys::check(unsafe { T::fx_conv2d_dgrad(Self::raw()?, self.hip_data.ptr(), f.hip_data.ptr(), out.ptr_mut(), &d, mode) })?;
        Self::boxed(out)
    }
    /// self is the convolution's input, other the upstream gradient, output_shape the filter's shape.
    fn cross_correlation2d(&self, other: &dyn StorageBackend<T>, output_shape: &[usize], stride: (usize, usize), padding: (usize, usize)) -> Boxed<T> {
        if self.shape().len() != 4 || other.shape().len() != 4 || output_shape.len() != 4 {
            return Err("Cross correlation requires 4D tensors [batch, channels, height, width]".to_string());
        }
        let g = Self::gpu(other, "Mixed GPU/CPU deconvolution not supported - move both tensors to same device")?;
        let d = Self::conv_dims(self.shape(), output_shape, stride, padding);
        let out = HipTensor::<T>::alloc(output_shape)?;
        let mode = hip_context()?.conv_grad_mode;
        sys::check(unsafe { T::fx_conv2d_wgrad(Self::raw()?, self.hip_data.ptr(), g.hip_data.ptr(), out.ptr_mut(), &d, mode) })?;
        Self::boxed(out)
    }
    // The 1-D convolutions of the reference work on plain vectors (a toy path outside the training step): not on this backend.
    fn conv1d(&self, _filter: &dyn StorageBackend<T>) -> Boxed<T> {
        Err("conv1d is not implemented on the HIP backend; move the tensors to the CPU".to_string())
    }
    fn deconv1d(&self, _filter: &dyn StorageBackend<T>) -> Boxed<T> {
        Err("deconv1d is not implemented on the HIP backend; move the tensors to the CPU".to_string())
    }
    fn cross_correlation1d(&self, _other: &dyn StorageBackend<T>) -> Boxed<T> {
        Err("cross_correlation1d is not implemented on the HIP backend; move the tensors to the CPU".to_string())
    }

    // ---- element access stays on the CPU (storage/cuda.rs:1024-1034) ----
    fn iter_values(&self) -> Result<Vec<T>, String> {
        Err("Cannot iterate over a tensor in cuda. Move to cpu first.".to_string())
    }
    fn get_flat(&self, _index: usize) -> Result<Option<T>, String> {
        Err("Cannot index over a tensor in cuda. Move to cpu first.".to_string())
    }
    fn get_multi(&self, _indices: &[usize]) -> Result<Option<T>, String> {
        Err("Cannot index over a tensor in cuda. Move to cpu first.".to_string())
    }

    // ---- pooling and its gradients (storage/cuda.rs:1127-1375); the 1-D calls are H = 1 with a 1 x k window ----
    fn maxpool2d(&self, kernel_size: usize, stride: usize, padding: usize) -> Boxed<T> {
        let s = self.shape();
        if s.len() != 4 {
            return Err("Maxpool2d requires 4D tensor [N, C, H, W]".to_string());
        }
        let (k, st, p) = (kernel_size, stride, padding);
        let d = [s[0] as i64, s[1] as i64, s[2] as i64, s[3] as i64, k as i64, k as i64, st as i64, st as i64, p as i64, p as i64];
        self.pool(true, d, &[s[0], s[1], (s[2] + 2 * p - k) / st + 1, (s[3] + 2 * p - k) / st + 1])
    }
    fn avgpool2d(&self, kernel_size: usize, stride: usize, padding: usize) -> Boxed<T> {
        let s = self.shape();
        if s.len() != 4 {
            return Err("Avgpool2d requires 4D tensor [N, C, H, W]".to_string());
        }
        let (k, st, p) = (kernel_size, stride, padding);
        let d = [s[0] as i64, s[1] as i64, s[2] as i64, s[3] as i64, k as i64, k as i64, st as i64, st as i64, p as i64, p as i64];
        self.pool(false, d, &[s[0], s[1], (s[2] + 2 * p - k) / st + 1, (s[3] + 2 * p - k) / st + 1])
    }
    fn maxpool1d(&self, kernel_size: usize, stride: usize, padding: usize) -> Boxed<T> {
        let s = self.shape();
        if s.len() != 3 {
            return Err("Maxpool1d requires 3D tensor [N, C, L]".to_string());
        }
        let (k, st, p) = (kernel_size, stride, padding);
        let d = [s[0] as i64, s[1] as i64, 1, s[2] as i64, 1, k as i64, 1, st as i64, 0, p as i64];
        self.pool(true, d, &[s[0], s[1], (s[2] + 2 * p - k) / st + 1])
    }
    fn avgpool1d(&self, kernel_size: usize, stride: usize, padding: usize) -> Boxed<T> {
        let s = self.shape();
        if s.len() != 3 {
            return Err("Avgpool1d requires 3D tensor [N, C, L]".to_string());
        }
        let (k, st, p) = (kernel_size, stride, padding);
        let d = [s[0] as i64, s[1] as i64, 1, s[2] as i64, 1, k as i64, 1, st as i64, 0, p as i64];
        self.pool(false, d, &[s[0], s[1], (s[2] + 2 * p - k) / st + 1])
    }
    fn max_unpool2d(&self, grad_output: &dyn StorageBackend<T>, original_input: &dyn StorageBackend<T>, pooled_output: &dyn StorageBackend<T>,
                    kernel_size: usize, stride: usize, padding: usize) -> Boxed<T> {
        Self::unpool(true, "max unpool2d", grad_output, original_input, pooled_output, (kernel_size, kernel_size), (stride, stride), (padding, padding))
    }
    fn avg_unpool2d(&self, grad_output: &dyn StorageBackend<T>, original_input: &dyn StorageBackend<T>, pooled_output: &dyn StorageBackend<T>,
                    kernel_size: usize, stride: usize, padding: usize) -> Boxed<T> {
        Self::unpool(false, "avg unpool2d", grad_output, original_input, pooled_output, (kernel_size, kernel_size), (stride, stride), (padding, padding))
    }
    fn max_unpool1d(&self, grad_output: &dyn StorageBackend<T>, original_input: &dyn StorageBackend<T>, pooled_output: &dyn StorageBackend<T>,
                    kernel_size: usize, stride: usize, padding: usize) -> Boxed<T> {
        Self::unpool(true, "max unpool1d", grad_output, original_input, pooled_output, (1, kernel_size), (1, stride), (0, padding))
    }
    fn avg_unpool1d(&self, grad_output: &dyn StorageBackend<T>, original_input: &dyn StorageBackend<T>, pooled_output: &dyn StorageBackend<T>,
                    kernel_size: usize, stride: usize, padding: usize) -> Boxed<T> {
        Self::unpool(false, "avg unpool1d", grad_output, original_input, pooled_output, (1, kernel_size), (1, stride), (0, padding))
    }
}
