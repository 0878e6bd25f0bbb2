//! GpuTensor (nn/tensor.rs:45-282): dense, row-major fp32 in device memory; `reshape` shares the storage.
use std::ffi::c_void;
use std::sync::Arc;

use agpu_sys as sys;

use crate::error::{NnError, Result};
use crate::registry::KernelRegistry;

struct Storage {
    reg: Arc<KernelRegistry>,
    ptr: *mut c_void,
}

impl Drop for Storage {
    fn drop(&mut self) {
        unsafe { sys::agpu_free(self.reg.raw(), self.ptr) };
    }
}

#[derive(Clone)]
pub struct GpuTensor {
    store: Arc<Storage>,
    shape: Vec<usize>,
}

impl GpuTensor {
    /// alloc_zeros of the reference's operators: a zeroed tensor of the given shape.
    pub fn zeros(shape: &[usize], reg: &Arc<KernelRegistry>) -> Result<GpuTensor> {
        let n: usize = shape.iter().product();
        let mut ptr: *mut c_void = std::ptr::null_mut();
        reg.check(unsafe { sys::agpu_malloc(reg.raw(), n.max(1) * 4, &mut ptr) })?;
        Ok(GpuTensor { store: Arc::new(Storage { reg: Arc::clone(reg), ptr }), shape: shape.to_vec() })
    }

    /// GpuTensor::from_host (tensor.rs:85-106): the data length must match the shape.
    pub fn from_host(data: &[f32], shape: &[usize], reg: &Arc<KernelRegistry>) -> Result<GpuTensor> {
        let n: usize = shape.iter().product();
        if data.len() != n {
            return Err(NnError::ShapeMismatch { expected: format!("{n} elements"), actual: format!("{} elements", data.len()) });
        }
        let t = GpuTensor::zeros(shape, reg)?;
        reg.check(unsafe { sys::agpu_memcpy_h2d(reg.raw(), t.store.ptr, data.as_ptr() as *const c_void, n * 4) })?;
        Ok(t)
    }

    pub fn to_host(&self) -> Result<Vec<f32>> {
        let mut out = vec![0f32; self.numel()];
        let reg = &self.store.reg;
        reg.check(unsafe { sys::agpu_memcpy_d2h(reg.raw(), out.as_mut_ptr() as *mut c_void, self.store.ptr, out.len() * 4) })?;
        Ok(out)
    }

    /// reshape (tensor.rs:201-222): same storage, new shape, same element count.
    pub fn reshape(&self, shape: &[usize]) -> Result<GpuTensor> {
        let n: usize = shape.iter().product();
        if n != self.numel() {
            return Err(NnError::ShapeMismatch { expected: format!("{} elements", self.numel()), actual: format!("{n} elements") });
        }
        Ok(GpuTensor { store: Arc::clone(&self.store), shape: shape.to_vec() })
    }

    /// clone_tensor (tensor.rs:270-282): a device-to-device copy.
    pub fn clone_tensor(&self) -> Result<GpuTensor> {
        let t = GpuTensor::zeros(&self.shape, &self.store.reg)?;
        let reg = &self.store.reg;
        reg.check(unsafe { sys::agpu_memcpy_d2d(reg.raw(), t.store.ptr, self.store.ptr, self.numel() * 4) })?;
        Ok(t)
    }

    pub fn shape(&self) -> &[usize] {
        &self.shape
    }
    pub fn ndim(&self) -> usize {
        self.shape.len()
    }
    pub fn dim(&self, i: usize) -> Result<usize> {
        self.shape.get(i).copied().ok_or(NnError::DimOutOfRange { dim: i, ndim: self.shape.len() })
    }
    pub fn numel(&self) -> usize {
        self.shape.iter().product()
    }
    /// Rows of a `[*, cols]` tensor (every leading dimension flattened, int4_linear.rs:81-90).
    pub fn rows(&self) -> usize {
        match self.shape.last() {
            Some(&c) if c > 0 => self.numel() / c,
            _ => 0,
        }
    }
    pub fn data(&self) -> *const f32 {
        self.store.ptr as *const f32
    }
    pub fn data_mut(&self) -> *mut f32 {
        self.store.ptr as *mut f32
    }
    pub fn registry(&self) -> &Arc<KernelRegistry> {
        &self.store.reg
    }
}
