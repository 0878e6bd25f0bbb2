//! GpuArray (gpu_array.rs:42-385): a host vector with a device copy made on demand and a residency state that says
//! which of the two is current.  Below 64 KiB the device side is pinned host memory that kernels access in place
//! (`agpu_host_alloc_mapped`, the reference's `MappedBuffer`); at or above it, device memory with explicit copies.
use std::cell::{Cell, UnsafeCell};
use std::ffi::c_void;
use std::ops::{Deref, DerefMut};
use std::sync::Arc;

use agpu_sys as sys;

use crate::error::Result;
use crate::registry::KernelRegistry;

/// SIZE_THRESHOLD_BYTES (gpu_array.rs:45-51).
const SIZE_THRESHOLD_BYTES: usize = 64 * 1024;

/// Residency (gpu_array.rs:55-69).
#[derive(Clone, Copy, PartialEq, Eq, Debug)]
pub enum Residency {
    HostOnly,
    Synced,
    DeviceOnly,
    HostDirty,
}

enum DeviceStorage {
    Mapped { host: *mut c_void, dev: *mut c_void, reg: Arc<KernelRegistry> },
    DeviceMem { dev: *mut c_void, reg: Arc<KernelRegistry> },
}

impl DeviceStorage {
    fn dev_ptr(&self) -> u64 {
        match self {
            DeviceStorage::Mapped { dev, .. } | DeviceStorage::DeviceMem { dev, .. } => *dev as u64,
        }
    }
}

impl Drop for DeviceStorage {
    fn drop(&mut self) {
        unsafe {
            match self {
                DeviceStorage::Mapped { host, reg, .. } => {
                    sys::agpu_host_free_mapped(reg.raw(), *host);
                }
                DeviceStorage::DeviceMem { dev, reg } => {
                    sys::agpu_free(reg.raw(), *dev);
                }
            }
        }
    }
}

pub struct GpuArray<T: Copy + Send + 'static> {
    host: UnsafeCell<Vec<T>>,
    device: UnsafeCell<Option<DeviceStorage>>,
    residency: Cell<Residency>,
    len: usize,
}

// Ownership may move between threads; shared access from two threads is not supported (Cell, UnsafeCell), as in the
// reference (gpu_array.rs:112-136).
unsafe impl<T: Copy + Send + 'static> Send for GpuArray<T> {}

impl<T: Copy + Send + 'static> GpuArray<T> {
    pub fn from_vec(data: Vec<T>) -> Self {
        let len = data.len();
        GpuArray { host: UnsafeCell::new(data), device: UnsafeCell::new(None), residency: Cell::new(Residency::HostOnly), len }
    }
    pub fn from_slice(data: &[T]) -> Self {
        Self::from_vec(data.to_vec())
    }
    pub fn len(&self) -> usize {
        self.len
    }
    pub fn is_empty(&self) -> bool {
        self.len == 0
    }
    pub fn residency(&self) -> Residency {
        self.residency.get()
    }
    pub fn should_use_mapped(&self) -> bool {
        self.len * std::mem::size_of::<T>() < SIZE_THRESHOLD_BYTES
    }
    fn bytes(&self) -> usize {
        self.len * std::mem::size_of::<T>()
    }

    /// Device-to-host sync (gpu_array.rs:178-218); the caller holds the only reference to the host data.
    fn sync_to_host_fallible(&self) -> Result<()> {
        let storage = unsafe { &*self.device.get() };
        let host = unsafe { &mut *self.host.get() };
        if let Some(st) = storage {
            match st {
                DeviceStorage::Mapped { host: mapped, reg, .. } => {
                    reg.synchronize()?; // the kernel that wrote the memory has finished
                    unsafe { std::ptr::copy_nonoverlapping(*mapped as *const T, host.as_mut_ptr(), self.len) };
                }
                DeviceStorage::DeviceMem { dev, reg } => {
                    reg.check(unsafe { sys::agpu_memcpy_d2h(reg.raw(), host.as_mut_ptr() as *mut c_void, *dev, self.bytes()) })?;
                }
            }
        }
        self.residency.set(Residency::Synced);
        Ok(())
    }

    /// try_sync_to_host (gpu_array.rs:208-225): the host data, with a sync error returned instead of a panic.
    pub fn try_sync_to_host(&self) -> Result<&[T]> {
        if self.residency.get() == Residency::DeviceOnly {
            self.sync_to_host_fallible()?;
        }
        Ok(unsafe { &*self.host.get() })
    }

    /// mark_device_dirty (gpu_array.rs:227-240): a kernel wrote the device copy.
    pub fn mark_device_dirty(&self) {
        if self.residency.get() == Residency::Synced {
            self.residency.set(Residency::DeviceOnly);
        }
    }

    /// ensure_device (gpu_array.rs:241-340): the device address of the data, uploaded if the host copy is newer.
    pub fn ensure_device(&self, reg: &Arc<KernelRegistry>) -> Result<u64> {
        match self.residency.get() {
            Residency::HostOnly => {
                if self.len == 0 {
                    self.residency.set(Residency::Synced);
                    return Ok(0);
                }
                let host = unsafe { &*self.host.get() };
                let storage = if self.should_use_mapped() {
                    let (mut h, mut d): (*mut c_void, *mut c_void) = (std::ptr::null_mut(), std::ptr::null_mut());
                    reg.check(unsafe { sys::agpu_host_alloc_mapped(reg.raw(), self.bytes(), &mut h, &mut d) })?;
                    unsafe { std::ptr::copy_nonoverlapping(host.as_ptr(), h as *mut T, self.len) };
                    DeviceStorage::Mapped { host: h, dev: d, reg: Arc::clone(reg) }
                } else {
                    let mut d: *mut c_void = std::ptr::null_mut();
                    reg.check(unsafe { sys::agpu_malloc(reg.raw(), self.bytes(), &mut d) })?;
                    let st = DeviceStorage::DeviceMem { dev: d, reg: Arc::clone(reg) };
                    reg.check(unsafe { sys::agpu_memcpy_h2d(reg.raw(), d, host.as_ptr() as *const c_void, self.bytes()) })?;
                    st
                };
                let ptr = storage.dev_ptr();
                unsafe { *self.device.get() = Some(storage) };
                self.residency.set(Residency::Synced);
                Ok(ptr)
            }
            Residency::HostDirty => {
                let host = unsafe { &*self.host.get() };
                let storage = unsafe { &*self.device.get() };
                match storage {
                    None => {
                        // modified before the first upload: nothing on the device yet
                        self.residency.set(Residency::HostOnly);
                        self.ensure_device(reg)
                    }
                    Some(st) => {
                        match st {
                            DeviceStorage::Mapped { host: mapped, reg, .. } => {
                                reg.synchronize()?; // no kernel may still be reading the old contents
                                unsafe { std::ptr::copy_nonoverlapping(host.as_ptr(), *mapped as *mut T, self.len) };
                            }
                            DeviceStorage::DeviceMem { dev, reg } => {
                                reg.check(unsafe { sys::agpu_memcpy_h2d(reg.raw(), *dev, host.as_ptr() as *const c_void, self.bytes()) })?;
                            }
                        }
                        self.residency.set(Residency::Synced);
                        Ok(st.dev_ptr())
                    }
                }
            }
            Residency::Synced | Residency::DeviceOnly => Ok(unsafe { &*self.device.get() }.as_ref().map(|s| s.dev_ptr()).unwrap_or(0)),
        }
    }
}

impl<T: Copy + Send + Default + 'static> GpuArray<T> {
    /// zeroed (gpu_array.rs:344-351)
    pub fn zeroed(len: usize) -> Self {
        Self::from_vec(vec![T::default(); len])
    }
}

impl<T: Copy + Send + 'static> Deref for GpuArray<T> {
    type Target = [T];
    fn deref(&self) -> &[T] {
        if self.residency.get() == Residency::DeviceOnly {
            self.sync_to_host_fallible().expect("GpuArray: device-to-host sync failed");
        }
        unsafe { &*self.host.get() }
    }
}

impl<T: Copy + Send + 'static> DerefMut for GpuArray<T> {
    fn deref_mut(&mut self) -> &mut [T] {
        if self.residency.get() == Residency::DeviceOnly {
            self.sync_to_host_fallible().expect("GpuArray: device-to-host sync failed");
        }
        self.residency.set(Residency::HostDirty);
        unsafe { &mut *self.host.get() }
    }
}

impl<T: Copy + Send + 'static> From<Vec<T>> for GpuArray<T> {
    fn from(data: Vec<T>) -> Self {
        Self::from_vec(data)
    }
}

impl<T: Copy + Send + 'static> From<&[T]> for GpuArray<T> {
    fn from(data: &[T]) -> Self {
        Self::from_slice(data)
    }
}

/// AsDevicePtr (gpu_array.rs:404-428): what a kernel launch needs of an argument.
pub trait AsDevicePtr {
    fn ensure_device(&self, reg: &Arc<KernelRegistry>) -> Result<u64>;
    fn device_len(&self) -> usize;
    fn mark_device_dirty(&self);
}

impl<T: Copy + Send + 'static> AsDevicePtr for GpuArray<T> {
    fn ensure_device(&self, reg: &Arc<KernelRegistry>) -> Result<u64> {
        GpuArray::ensure_device(self, reg)
    }
    fn device_len(&self) -> usize {
        self.len
    }
    fn mark_device_dirty(&self) {
        GpuArray::mark_device_dirty(self)
    }
}

#[cfg(test)]
mod tests {
    use super::*;

    // The host-only life cycle, as the reference tests it (gpu_array.rs:434-514).
    #[test]
    fn from_vec_creates_host_only() {
        let arr = GpuArray::from_vec(vec![1.0f32, 2.0, 3.0]);
        assert_eq!(arr.residency(), Residency::HostOnly);
        assert_eq!(arr.len(), 3);
        assert!(!arr.is_empty());
    }

    #[test]
    fn deref_mut_marks_host_dirty() {
        let mut arr = GpuArray::from_vec(vec![1.0f32, 2.0, 3.0]);
        arr[0] = 99.0;
        assert_eq!(arr.residency(), Residency::HostDirty);
        assert_eq!(arr[0], 99.0);
    }

    #[test]
    fn size_thresholds() {
        assert!(GpuArray::from_vec(vec![0.0f32; 100]).should_use_mapped());
        assert!(!GpuArray::from_vec(vec![0.0f32; 16384]).should_use_mapped());
        assert!(GpuArray::from_vec(vec![0.0f32; 16383]).should_use_mapped());
    }

    #[test]
    fn empty_and_zeroed() {
        let arr = GpuArray::<f32>::from_vec(vec![]);
        assert!(arr.is_empty());
        let z = GpuArray::<f32>::zeroed(100);
        assert!(z.iter().all(|&x| x == 0.0));
    }
}
