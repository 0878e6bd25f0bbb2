//! KernelRegistry (nn/registry.rs:26-144): the handle every operator takes.  In the reference it owns the loaded PTX
//! module and hands out `CudaFunction`s by name; here it owns the context of libagpu_hip.so (device, stream,
//! scratch) and answers `get(name)` with the entry point that serves the reference's kernel name.
use std::ffi::{CStr, CString};
use std::sync::Arc;

use agpu_sys as sys;

use crate::error::{NnError, Result};

pub struct KernelRegistry {
    ctx: *mut sys::agpu_ctx,
}

// One thread at a time uses a context (a second one is turned away with AGPU_ERR_BUSY); the handle itself may move.
unsafe impl Send for KernelRegistry {}
unsafe impl Sync for KernelRegistry {}

impl KernelRegistry {
    /// KernelRegistry::init_default (registry.rs:131-135): device 0 and its own stream.
    pub fn init_default() -> Result<Arc<KernelRegistry>> {
        Self::new(0)
    }

    pub fn new(device: i32) -> Result<Arc<KernelRegistry>> {
        let mut ctx: *mut sys::agpu_ctx = std::ptr::null_mut();
        let rc = unsafe { sys::agpu_ctx_create(device, &mut ctx) };
        if rc != sys::AGPU_OK {
            return Err(NnError::from_code(rc, "agpu_ctx_create failed".to_string()));
        }
        Ok(Arc::new(KernelRegistry { ctx }))
    }

    /// registry.get(name) (registry.rs:140-144): the C entry point serving one of the reference's kernel names.
    pub fn get(&self, name: &str) -> Result<String> {
        let c = CString::new(name).map_err(|_| NnError::KernelNotFound { name: name.to_string() })?;
        let mut entry: *const std::os::raw::c_char = std::ptr::null();
        let rc = unsafe { sys::agpu_kernel_lookup(self.ctx, c.as_ptr(), &mut entry) };
        if rc != sys::AGPU_OK || entry.is_null() {
            return Err(NnError::KernelNotFound { name: name.to_string() });
        }
        Ok(unsafe { CStr::from_ptr(entry) }.to_string_lossy().into_owned())
    }

    pub fn raw(&self) -> *mut sys::agpu_ctx {
        self.ctx
    }

    /// dev.synchronize()
    pub fn synchronize(&self) -> Result<()> {
        self.check(unsafe { sys::agpu_sync(self.ctx) })
    }

    /// Turns a return code into a `Result`, with the context's message.
    pub fn check(&self, rc: i32) -> Result<()> {
        if rc == sys::AGPU_OK {
            return Ok(());
        }
        let msg = unsafe { CStr::from_ptr(sys::agpu_last_error_string(self.ctx)) }.to_string_lossy().into_owned();
        Err(NnError::from_code(rc, msg))
    }
}

impl Drop for KernelRegistry {
    fn drop(&mut self) {
        // models created on the context keep its memory alive until they are gone too
        unsafe { sys::agpu_ctx_destroy(self.ctx) };
    }
}
