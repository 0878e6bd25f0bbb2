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

/// Where the device side of an array lives: `dev` is what kernels are given; `alias` is the same bytes as the host sees
/// them when the memory is pinned and mapped (small arrays), null when it is device memory that needs explicit copies.
struct Backing {
    dev: *mut c_void,
    alias: *mut c_void,
    bytes: usize,
    reg: Arc<KernelRegistry>,
}

impl Backing {
    fn create(reg: &Arc<KernelRegistry>, bytes: usize, mapped: bool) -> Result<Backing> {
        let (mut alias, mut dev): (*mut c_void, *mut c_void) = (std::ptr::null_mut(), std::ptr::null_mut());
        if mapped {
            reg.check(unsafe { sys::agpu_host_alloc_mapped(reg.raw(), bytes, &mut alias, &mut dev) })?;
        } else {
            reg.check(unsafe { sys::agpu_malloc(reg.raw(), bytes, &mut dev) })?;
        }
        Ok(Backing { dev, alias, bytes, reg: Arc::clone(reg) })
    }

    /// Host bytes to the device side.  Mapped memory is written in place once nothing on the stream can still be reading it.
    fn push(&self, src: *const c_void) -> Result<()> {
        if self.alias.is_null() {
            return self.reg.check(unsafe { sys::agpu_memcpy_h2d(self.reg.raw(), self.dev, src, self.bytes) });
        }
        self.reg.synchronize()?;
        unsafe { std::ptr::copy_nonoverlapping(src as *const u8, self.alias as *mut u8, self.bytes) };
        Ok(())
    }

    /// The device side back into host bytes, once the kernels that wrote it have finished.
    fn pull(&self, dst: *mut c_void) -> Result<()> {
        if self.alias.is_null() {
            return self.reg.check(unsafe { sys::agpu_memcpy_d2h(self.reg.raw(), dst, self.dev, self.bytes) });
        }
        self.reg.synchronize()?;
        unsafe { std::ptr::copy_nonoverlapping(self.alias as *const u8, dst as *mut u8, self.bytes) };
        Ok(())
    }
}

impl Drop for Backing {
    fn drop(&mut self) {
        unsafe {
            if self.alias.is_null() {
                sys::agpu_free(self.reg.raw(), self.dev);
            } else {
                sys::agpu_host_free_mapped(self.reg.raw(), self.alias);
            }
        }
    }
}

pub struct GpuArray<T: Copy + Send + 'static> {
    elems: UnsafeCell<Vec<T>>,
    backing: UnsafeCell<Option<Backing>>,
    state: Cell<Residency>,
}

// Ownership may move between threads; shared access from two threads is not supported (Cell, UnsafeCell), as in the
// reference (gpu_array.rs:112-136).
unsafe impl<T: Copy + Send + 'static> Send for GpuArray<T> {}

impl<T: Copy + Send + 'static> GpuArray<T> {
    pub fn from_vec(data: Vec<T>) -> Self {
        GpuArray { elems: UnsafeCell::new(data), backing: UnsafeCell::new(None), state: Cell::new(Residency::HostOnly) }
    }
    pub fn from_slice(data: &[T]) -> Self {
        Self::from_vec(data.to_vec())
    }
    pub fn len(&self) -> usize {
        self.host().len()
    }
    pub fn is_empty(&self) -> bool {
        self.len() == 0
    }
    pub fn residency(&self) -> Residency {
        self.state.get()
    }
    pub fn should_use_mapped(&self) -> bool {
        self.bytes() < SIZE_THRESHOLD_BYTES
    }
    fn bytes(&self) -> usize {
        self.len() * std::mem::size_of::<T>()
    }
    fn host(&self) -> &Vec<T> {
        unsafe { &*self.elems.get() }
    }
    fn backing(&self) -> Option<&Backing> {
        unsafe { &*self.backing.get() }.as_ref()
    }

    /// The one place where copies happen.  `newer_on_device` false: make the device side current (creating it on first
    /// use) and return its address; true: make the host side current.  Either way the array ends up Synced.
    fn reconcile(&self, reg: Option<&Arc<KernelRegistry>>, newer_on_device: bool) -> Result<u64> {
        if newer_on_device {
            if let Some(b) = self.backing() {
                b.pull(unsafe { &mut *self.elems.get() }.as_mut_ptr() as *mut c_void)?;
            }
            self.state.set(Residency::Synced);
            return Ok(self.backing().map(|b| b.dev as u64).unwrap_or(0));
        }
        if self.is_empty() {
            self.state.set(Residency::Synced);
            return Ok(0);
        }
        if self.backing().is_none() {
            let reg = reg.expect("GpuArray: no registry to create the device side with");
            let made = Backing::create(reg, self.bytes(), self.should_use_mapped())?;
            unsafe { *self.backing.get() = Some(made) };
        }
        let b = self.backing().unwrap();
        b.push(self.host().as_ptr() as *const c_void)?;
        self.state.set(Residency::Synced);
        Ok(b.dev as u64)
    }

    /// try_sync_to_host (gpu_array.rs:208-225): the host data, with a sync error returned instead of a panic.
    pub fn try_sync_to_host(&self) -> Result<&[T]> {
        if self.state.get() == Residency::DeviceOnly {
            self.reconcile(None, true)?;
        }
        Ok(self.host())
    }

    /// mark_device_dirty (gpu_array.rs:227-240): a kernel wrote the device copy.
    pub fn mark_device_dirty(&self) {
        if self.state.get() == Residency::Synced {
            self.state.set(Residency::DeviceOnly);
        }
    }

    /// ensure_device (gpu_array.rs:241-340): the device address of the data, uploaded if the host copy is newer
    /// (HostOnly: first upload; HostDirty: the host was written since the last one).
    pub fn ensure_device(&self, reg: &Arc<KernelRegistry>) -> Result<u64> {
        match self.state.get() {
            Residency::HostOnly | Residency::HostDirty => self.reconcile(Some(reg), false),
            Residency::Synced | Residency::DeviceOnly => Ok(self.backing().map(|b| b.dev as u64).unwrap_or(0)),
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
        if self.state.get() == Residency::DeviceOnly {
            self.reconcile(None, true).expect("GpuArray: device-to-host sync failed");
        }
        self.host()
    }
}

impl<T: Copy + Send + 'static> DerefMut for GpuArray<T> {
    fn deref_mut(&mut self) -> &mut [T] {
        if self.state.get() == Residency::DeviceOnly {
            self.reconcile(None, true).expect("GpuArray: device-to-host sync failed");
        }
        self.state.set(Residency::HostDirty);
        self.elems.get_mut().as_mut_slice()
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
        self.len()
    }
    fn mark_device_dirty(&self) {
        GpuArray::mark_device_dirty(self)
    }
}

#[cfg(test)]
mod host_side {
    use super::{GpuArray, Residency};

    // What can be checked without a device: the states a host-only array goes through (the reference checks the same
    // properties in gpu_array.rs:434-514), and on which side of 64 KiB an array falls.
    #[test]
    fn a_fresh_array_lives_on_the_host() {
        let a = GpuArray::from_slice(&[4u32, 5, 6, 7]);
        assert!(a.residency() == Residency::HostOnly && a.len() == 4 && !a.is_empty());
        assert_eq!(&a[..], &[4, 5, 6, 7]);
    }

    #[test]
    fn writing_through_the_array_makes_the_host_newer() {
        let mut a: GpuArray<f64> = vec![0.5, 1.5].into();
        a[1] = -2.0;
        assert!(a.residency() == Residency::HostDirty);
        assert_eq!(a.try_sync_to_host().unwrap(), &[0.5, -2.0]);
    }

    #[test]
    fn sixty_four_kib_is_the_first_size_in_device_memory() {
        for (n, mapped) in [(1usize, true), (16383, true), (16384, false), (100_000, false)] {
            assert_eq!(GpuArray::<f32>::zeroed(n).should_use_mapped(), mapped, "{n} floats");
        }
    }

    #[test]
    fn an_empty_array_is_empty() {
        assert!(GpuArray::<u8>::from_vec(Vec::new()).is_empty());
        assert!(GpuArray::<i32>::zeroed(9).iter().all(|&v| v == 0));
    }
}
